// Member lists of the clusters: rows sorted by cluster id, ties in ascending row order.
//
// The sort is a stable LSD radix sort written for this job (8-bit digits, keys of at most 30
// bits, the row number as payload): per pass a digit histogram per tile of 4,096 keys, a scan
// of the histograms, and a scatter that ranks the keys of a tile in index order with wave
// ballots, so the order of equal keys is kept without any atomic on global memory.  The first
// pass takes the row numbers from the positions (no index array is written or read first).
// It runs once per assignment refresh, not per training step.
//
// cgnn_lsh_group derives ids, counts and member lists from the raw hash codes with that sort:
// the dense id of a row is the rank of its code among the codes that occur, so sorting by code
// is sorting by id, the groups are the runs of equal codes and no counter is ever updated
// atomically (rows of a graph pile up in a few codes).  With at most 16 hyperplanes the ranks
// come from a table over all codes (which codes occur, scanned), so the ids are written in row
// order with coalesced stores; with more hyperplanes from a scan over the sorted rows.
#include <algorithm>

#include "common.h"
#include "radix_sort.h"

namespace cgnn {
namespace {

// ------------------------------------------------------------------- radix sort --
constexpr int kDigitBits = 8;
constexpr int kDigits = 1 << kDigitBits;           // one per thread of a workgroup
constexpr int kSortItems = 16;                     // keys per thread
constexpr int kSortTile = kBlock * kSortItems;     // keys per workgroup
static_assert(kDigits == kBlock, "one digit per thread");

__device__ __forceinline__ int digit_of(int32_t key, int shift) { return (key >> shift) & (kDigits - 1); }

// hist[d * tiles + tile] = number of keys of the tile with digit d (digit-major: the scan over a
// digit's tiles is a scan over consecutive entries).  THREADS: the workgroup's size, a multiple
// of kDigits; the loads of a thread are all issued before the first count.
template <int THREADS>
__device__ __forceinline__ void tile_histogram(const int32_t *__restrict__ keys, int64_t N, int shift,
                                               int32_t *__restrict__ hist, int tiles, int tile, int *count) {
    constexpr int kItems = kSortTile / THREADS;
    if (threadIdx.x < kDigits) count[threadIdx.x] = 0;
    __syncthreads();
    const int64_t base = (int64_t)tile * kSortTile;
    int32_t key[kItems];
#pragma unroll
    for (int it = 0; it < kItems; ++it) {
        const int64_t i = base + (int64_t)it * THREADS + threadIdx.x;
        key[it] = i < N ? keys[i] : 0;
    }
#pragma unroll
    for (int it = 0; it < kItems; ++it) {
        const int64_t i = base + (int64_t)it * THREADS + threadIdx.x;
        if (i < N) atomicAdd(&count[digit_of(key[it], shift)], 1);  // LDS, integer: the sum does not depend on the order
    }
    __syncthreads();
    if (threadIdx.x < kDigits) hist[(int64_t)threadIdx.x * tiles + tile] = count[threadIdx.x];
}

// `clear` (optional, first pass): a table of clear_n entries that this launch sets to zero, for
// the scatter of the same pass to mark.
__global__ __launch_bounds__(kBlock) void radix_hist_kernel(const int32_t *__restrict__ keys, int64_t N, int shift,
                                                           int32_t *__restrict__ hist, int tiles,
                                                           int32_t *__restrict__ clear, int clear_n) {
    __shared__ int count[kDigits];
    if (clear)
        for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < clear_n; i += (int64_t)gridDim.x * kBlock)
            clear[i] = 0;
    tile_histogram<kBlock>(keys, N, shift, hist, tiles, blockIdx.x, count);
}

// One wave per digit: within[d * tiles + t] = keys with digit d in the tiles before t, and
// total[d] = keys with digit d.
__global__ __launch_bounds__(kBlock) void radix_scan_kernel(const int32_t *__restrict__ hist, int tiles,
                                                           int32_t *__restrict__ within, int32_t *__restrict__ total) {
    const int lane = threadIdx.x % kWave;
    const int d = blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
    if (d >= kDigits) return;
    const int32_t *row = hist + (int64_t)d * tiles;
    int32_t *out = within + (int64_t)d * tiles;
    int running = 0;
    for (int t0 = 0; t0 < tiles; t0 += kWave) {
        const int t = t0 + lane;
        const int v = t < tiles ? row[t] : 0;
        int inc = v;
#pragma unroll
        for (int s = 1; s < kWave; s <<= 1) {
            const int n = __shfl_up(inc, s, kWave);
            if (lane >= s) inc += n;
        }
        if (t < tiles) out[t] = running + inc - v;
        running += __shfl(inc, kWave - 1, kWave);
    }
    if (lane == 0) total[d] = running;
}

// Lanes of the wave (among `active`) whose digit equals this lane's.
__device__ __forceinline__ unsigned long long same_digit(int d, unsigned long long active) {
    unsigned long long peers = active;
#pragma unroll
    for (int b = 0; b < kDigitBits; ++b) {
        const unsigned long long m = __ballot((d >> b) & 1);
        peers &= ((d >> b) & 1) ? m : ~m;
    }
    return peers;
}

// Scatter of one tile.  Wave w takes the w-th quarter of the tile, 64 consecutive keys per
// step, so "earlier in the tile" is "in an earlier wave, an earlier step of the same wave, or
// a lower lane of the same step": the rank of a key among the keys of its digit in the tile
// is counted in exactly that order, which keeps the sort stable.  The tile is first put in
// order in LDS and then written out position by position, so that neighbouring threads store
// to neighbouring addresses wherever a digit holds more than one key of the tile.
// vals == NULL: the payload of key i is i.  `seen` (optional): seen[key & seen_mask] = 1 for
// every key, the table the dense ranks of the hash codes are made from (the mask keeps a code
// beyond the table, a caller's mistake, inside it).  `remap` (optional, last pass): the keys are
// written as remap[key & seen_mask], an order-preserving renaming (the rank of the code).
__global__ __launch_bounds__(kBlock) void radix_scatter_kernel(const int32_t *__restrict__ keys,
                                                              const int32_t *__restrict__ vals, int64_t N, int shift,
                                                              const int32_t *__restrict__ within,
                                                              const int32_t *__restrict__ total, int tiles,
                                                              int32_t *__restrict__ keys_out,
                                                              int32_t *__restrict__ vals_out,
                                                              int32_t *__restrict__ seen, int seen_mask,
                                                              const int32_t *__restrict__ remap) {
    constexpr int kWaves = kBlock / kWave;
    constexpr int kPerWave = kSortTile / kWaves;
    __shared__ int digit_start[kDigits];         // output position of the tile's first key of a digit, minus tile_start
    __shared__ int tile_start[kDigits];          // position of that key in the ordered tile
    __shared__ int wave_count[kWaves][kDigits];  // keys of a digit seen by a wave so far; then: by the waves before it
    __shared__ int scan_tmp[2][kWaves];
    __shared__ int32_t tile_key[kSortTile], tile_val[kSortTile];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int mine = total[threadIdx.x];  // thread = digit
    const int my_within = within[(int64_t)threadIdx.x * tiles + blockIdx.x];
#pragma unroll
    for (int w = 0; w < kWaves; ++w) wave_count[w][threadIdx.x] = 0;
    __syncthreads();
    const int64_t base = (int64_t)blockIdx.x * kSortTile + (int64_t)wave * kPerWave;
    int32_t key[kSortItems], val[kSortItems];
    int rank[kSortItems];
    const unsigned long long below = (1ull << lane) - 1ull;
#pragma unroll
    for (int it = 0; it < kSortItems; ++it) {
        const int64_t i = base + (int64_t)it * kWave + lane;
        const bool live = i < N;
        key[it] = live ? keys[i] : 0;
        val[it] = live ? (vals ? vals[i] : (int32_t)i) : 0;
    }
#pragma unroll
    for (int it = 0; it < kSortItems; ++it) {
        const int64_t i = base + (int64_t)it * kWave + lane;
        const bool live = i < N;
        const int d = digit_of(key[it], shift);
        const unsigned long long peers = same_digit(d, __ballot(live));
        if (live) {
            const int seen_before = wave_count[wave][d];  // the same for all peers: read before any of them writes
            rank[it] = seen_before + __popcll(peers & below);
            if ((peers & below) == 0) wave_count[wave][d] = seen_before + __popcll(peers);
            if (seen) seen[key[it] & seen_mask] = 1;  // every writer stores the same value
        } else {
            rank[it] = 0;
        }
        __builtin_amdgcn_wave_barrier();  // the count written in this step is read in the next
    }
    __syncthreads();
    {   // per digit (thread = digit): what the waves before a wave hold, and the tile's count
        int running = 0;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            const int c = wave_count[w][threadIdx.x];
            wave_count[w][threadIdx.x] = running;
            running += c;
        }
        // exclusive scans over the digits: of the tile's counts (places in the ordered tile) and of
        // the totals (places in the output)
        int inc_tile = running, inc_all = mine;
#pragma unroll
        for (int s = 1; s < kWave; s <<= 1) {
            const int a = __shfl_up(inc_tile, s, kWave), b = __shfl_up(inc_all, s, kWave);
            if (lane >= s) {
                inc_tile += a;
                inc_all += b;
            }
        }
        if (lane == kWave - 1) {
            scan_tmp[0][wave] = inc_tile;
            scan_tmp[1][wave] = inc_all;
        }
        __syncthreads();
        int before_tile = 0, before_all = 0;
#pragma unroll
        for (int w = 0; w < kWaves; ++w)
            if (w < wave) {
                before_tile += scan_tmp[0][w];
                before_all += scan_tmp[1][w];
            }
        const int in_tile = before_tile + inc_tile - running;
        tile_start[threadIdx.x] = in_tile;
        digit_start[threadIdx.x] = before_all + inc_all - mine + my_within - in_tile;
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < kSortItems; ++it) {
        const int64_t i = base + (int64_t)it * kWave + lane;
        if (i < N) {
            const int d = digit_of(key[it], shift);
            const int at = tile_start[d] + wave_count[wave][d] + rank[it];
            tile_key[at] = key[it];
            tile_val[at] = val[it];
        }
    }
    __syncthreads();
    const int64_t left = N - (int64_t)blockIdx.x * kSortTile;
    const int in_this_tile = left < kSortTile ? (int)left : kSortTile;
#pragma unroll
    for (int it = 0; it < kSortItems; ++it) {
        const int at = it * kBlock + threadIdx.x;
        if (at < in_this_tile) {
            const int32_t k = tile_key[at];
            const int64_t pos = (int64_t)digit_start[digit_of(k, shift)] + at;
            keys_out[pos] = remap ? remap[k & seen_mask] : k;
            vals_out[pos] = tile_val[at];
        }
    }
}

int radix_passes(int bits) { return bits <= kDigitBits ? 1 : (bits + kDigitBits - 1) / kDigitBits; }
int64_t radix_tiles(int64_t N) { return ceil_div(N < 1 ? 1 : N, kSortTile); }

// hist, within (kDigits x tiles each) and total (kDigits)
size_t radix_counter_bytes(int64_t N) {
    return 2 * align_up((size_t)kDigits * (size_t)radix_tiles(N) * sizeof(int32_t), 256) + align_up(kDigits * sizeof(int32_t), 256);
}

// ------------------------------------------------------------------ member lists --
// An id outside [0, groups) is filed under the nearest group that exists (the lists then
// index nothing beyond their arrays) and reported through the flag.
__global__ void members_keys_kernel(const int64_t *__restrict__ ids, int32_t *__restrict__ keys, int64_t N,
                                    int64_t groups, int32_t *__restrict__ bad_id) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < N;
         i += (int64_t)gridDim.x * blockDim.x) {
        int64_t id = ids[i];
        if (id < 0 || id >= groups) {
            id = id < 0 ? 0 : groups - 1;
            if (bad_id) *bad_id = 1;  // every writer stores the same value
        }
        keys[i] = (int32_t)id;
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

// ------------------------------------------------- groups of equal hash codes ----
// More than 16 hyperplanes: head[p] = 1 where a run of equal codes starts.
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

// At most 16 hyperplanes: the table seen[code] (1 where the code occurs) becomes rank[code],
// the 1-based id of the code; summary[0] = number of codes that occur, summary[1] = 0 (the
// running maximum of the group sizes).  A workgroup ranks a stretch of 4,096 codes, four per
// thread, and counts for itself the codes that occur before its stretch (the table is 256 KB
// at most, so reading it again costs less than a second launch would); all loads of a thread
// are in flight together.
constexpr int kRankThreads = 1024;
constexpr int kRankStretch = 4 * kRankThreads;
constexpr int kTableBits = 16;  // up to this many hyperplanes the ranks come from a table over all codes
constexpr int kRankStretches = (1 << kTableBits) / kRankStretch;

__device__ __forceinline__ int occurs4(const int4 &v) { return (v.x != 0) + (v.y != 0) + (v.z != 0) + (v.w != 0); }

constexpr int kRankWaves = kRankThreads / kWave;

// stretch `part` of `parts`
__device__ __forceinline__ void code_rank_stretch(int32_t *__restrict__ table, int codes, int32_t *__restrict__ summary,
                                                  int part, int parts, int *wave_before, int *wave_mine) {
    constexpr int kWaves = kRankWaves;
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int4 *table4 = reinterpret_cast<const int4 *>(table);  // codes is a power of two: whole int4s from 4 codes on
    const int4 zero = {0, 0, 0, 0};
    const int quads = (codes + 3) / 4;
    // the stretches before this one, one int4 per thread and stretch
    int4 earlier[kRankStretches - 1];
#pragma unroll
    for (int k = 0; k < kRankStretches - 1; ++k) {
        const int q = k * kRankThreads + threadIdx.x;
        earlier[k] = (k < part && q < quads && codes >= 4) ? table4[q] : zero;
    }
    const int q = part * kRankThreads + threadIdx.x;
    int4 own = zero;
    if (codes >= 4) {
        if (q < quads) own = table4[q];
    } else if (q == 0) {  // one or two codes
        own.x = table[0];
        own.y = codes > 1 ? table[1] : 0;
    }
    int before = 0;
#pragma unroll
    for (int k = 0; k < kRankStretches - 1; ++k) before += occurs4(earlier[k]);
    const int mine = occurs4(own);
    // workgroup totals of `before`, exclusive scan of `mine`
    int sum_before = before, inc = mine;
#pragma unroll
    for (int s = 1; s < kWave; s <<= 1) {
        const int n = __shfl_up(inc, s, kWave);
        if (lane >= s) inc += n;
        sum_before += __shfl_xor(sum_before, s, kWave);
    }
    if (lane == kWave - 1) wave_mine[wave] = inc;
    if (lane == 0) wave_before[wave] = sum_before;
    __syncthreads();
    int running = 0, stretch_total = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
        running += wave_before[w];
        if (w < wave) running += wave_mine[w];
        stretch_total += wave_before[w] + wave_mine[w];
    }
    running += inc - mine;  // codes that occur before this thread's four
    int4 out;
    out.x = own.x != 0 ? ++running : 0;
    out.y = own.y != 0 ? ++running : 0;
    out.z = own.z != 0 ? ++running : 0;
    out.w = own.w != 0 ? ++running : 0;
    if (codes >= 4) {
        if (q < quads) reinterpret_cast<int4 *>(table)[q] = out;
    } else if (q == 0) {
        table[0] = out.x;
        if (codes > 1) table[1] = out.y;
    }
    if (part == parts - 1 && threadIdx.x == 0) {
        summary[0] = stretch_total;
        summary[1] = 0;
    }
}

__global__ __launch_bounds__(kRankThreads) void code_rank_kernel(int32_t *__restrict__ table, int codes,
                                                                 int32_t *__restrict__ summary) {
    __shared__ int wave_before[kRankWaves], wave_mine[kRankWaves];
    code_rank_stretch(table, codes, summary, blockIdx.x, gridDim.x, wave_before, wave_mine);
}

// The histograms of a later pass and the ranks of the codes in one launch: neither needs the
// other, both need the scatter of the first pass (its keys; the codes it has marked), and the
// sixteen workgroups of the ranks are over before the histograms are.
__global__ __launch_bounds__(kRankThreads) void radix_hist_rank_kernel(const int32_t *__restrict__ keys, int64_t N,
                                                                       int shift, int32_t *__restrict__ hist, int tiles,
                                                                       int32_t *__restrict__ table, int codes,
                                                                       int32_t *__restrict__ summary) {
    __shared__ int count[kDigits];
    __shared__ int wave_before[kRankWaves], wave_mine[kRankWaves];
    const int parts = (int)gridDim.x - tiles;
    if ((int)blockIdx.x < parts)  // first, so that they are not the tail of the launch
        code_rank_stretch(table, codes, summary, blockIdx.x, parts, wave_before, wave_mine);
    else
        tile_histogram<kRankThreads>(keys, N, shift, hist, tiles, (int)blockIdx.x - parts, count);
}

// Stable sort of (keys[i], i) by the low `bits` bits of the keys into (keys_out, vals_out).
// tmp_keys / tmp_vals: N entries each, used when there is more than one pass.  counters:
// radix_counter_bytes(N).  table (optional): seen_mask + 1 entries (a power of two); the first
// pass clears it and marks every key that occurs, code_rank_stretch (a launch of its own after
// a single pass, else part of the second pass's histogram launch) then turns it into the ranks
// of the keys (summary as there), and with more than one pass the last pass writes the ranks
// in place of the keys (*ranked = true).
int radix_sort_by_key(const int32_t *keys, int64_t N, int bits, int32_t *keys_out, int32_t *vals_out, int32_t *tmp_keys,
                      int32_t *tmp_vals, void *counters, int32_t *table, int seen_mask, int32_t *summary, bool *ranked,
                      hipStream_t stream) {
    if (ranked) *ranked = false;
    if (N <= 0) return CGNN_OK;
    const int passes = radix_passes(bits);
    const int tiles = (int)radix_tiles(N);
    char *cbase = static_cast<char *>(counters);
    const size_t tbytes = align_up((size_t)kDigits * (size_t)tiles * sizeof(int32_t), 256);
    int32_t *hist = reinterpret_cast<int32_t *>(cbase);
    int32_t *within = reinterpret_cast<int32_t *>(cbase + tbytes);
    int32_t *total = reinterpret_cast<int32_t *>(cbase + 2 * tbytes);
    const int32_t *in_keys = keys, *in_vals = nullptr;
    for (int p = 0; p < passes; ++p) {
        // the last pass writes the result; the passes before it alternate so that it can
        const bool to_result = (passes - 1 - p) % 2 == 0;
        int32_t *out_keys = to_result ? keys_out : tmp_keys, *out_vals = to_result ? vals_out : tmp_vals;
        const int shift = p * kDigitBits;
        const bool first = p == 0, last = p == passes - 1;
        const int32_t *remap = (table && last && !first) ? table : nullptr;
        const int rank_parts = (int)ceil_div(seen_mask + 1, kRankStretch);
        const bool rank_here = table && p == 1;  // the marks are complete after the first scatter
        if (rank_here)
            hipLaunchKernelGGL(radix_hist_rank_kernel, dim3((unsigned)(tiles + rank_parts)), dim3(kRankThreads), 0,
                               stream, in_keys, N, shift, hist, tiles, table, seen_mask + 1, summary);
        else
            hipLaunchKernelGGL(radix_hist_kernel, dim3((unsigned)tiles), dim3(kBlock), 0, stream, in_keys, N, shift,
                               hist, tiles, first ? table : nullptr, seen_mask + 1);
        hipLaunchKernelGGL(radix_scan_kernel, dim3(kDigits / (kBlock / kWave)), dim3(kBlock), 0, stream, hist, tiles,
                           within, total);
        hipLaunchKernelGGL(radix_scatter_kernel, dim3((unsigned)tiles), dim3(kBlock), 0, stream, in_keys, in_vals, N,
                           shift, within, total, tiles, out_keys, out_vals, first ? table : nullptr, seen_mask, remap);
        if (table && first && last)  // with a second pass its histogram launch makes the ranks
            hipLaunchKernelGGL(code_rank_kernel, dim3((unsigned)rank_parts), dim3(kRankThreads), 0, stream, table,
                               seen_mask + 1, summary);
        if (remap && ranked) *ranked = true;
        in_keys = out_keys;
        in_vals = out_vals;
    }
    return check_launch("radix_sort");
}

// The rest of an assignment from the rank table: ids in row order; in sorted order the id of
// every position (unless the sort has written the ranks already: `ranked`, and `sorted` is
// sorted_id itself) and the start of every group.
__global__ __launch_bounds__(kBlock) void group_table_finish_kernel(int64_t N, const int32_t *__restrict__ raw_code,
                                                                   const int32_t *sorted,
                                                                   const int32_t *__restrict__ rank, int code_mask,
                                                                   bool ranked, int64_t *__restrict__ ids,
                                                                   int32_t *sorted_id, int32_t *__restrict__ offsets) {
    // four positions a thread, a launch-wide stride apart: their loads are in flight together
    constexpr int kFinishItems = 4;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t p0 = (int64_t)blockIdx.x * kBlock + threadIdx.x; p0 < N; p0 += kFinishItems * stride) {
        int32_t code[kFinishItems], here[kFinishItems], before[kFinishItems];
#pragma unroll
        for (int u = 0; u < kFinishItems; ++u) {
            const int64_t p = p0 + u * stride;
            const bool live = p < N;
            code[u] = live ? raw_code[p] : 0;
            here[u] = live ? sorted[p] : 0;
            before[u] = live && p > 0 ? sorted[p - 1] : 0;
        }
        int32_t own_id[kFinishItems], id[kFinishItems];
#pragma unroll
        for (int u = 0; u < kFinishItems; ++u) {
            own_id[u] = rank[code[u] & code_mask];
            id[u] = ranked ? here[u] : rank[here[u] & code_mask];
        }
#pragma unroll
        for (int u = 0; u < kFinishItems; ++u) {
            const int64_t p = p0 + u * stride;
            if (p >= N) continue;
            ids[p] = own_id[u];
            if (!ranked) sorted_id[p] = id[u];
            if (p == 0) {
                offsets[0] = 0;
                offsets[id[u]] = 0;
            } else if (here[u] != before[u]) {  // codes and their ranks change at the same places
                offsets[id[u]] = (int32_t)p;
            }
            if (p == N - 1) offsets[id[u] + 1] = (int32_t)N;
        }
    }
}

// summary[0] = number of groups, summary[1] = largest group (cleared before this kernel).
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
    __shared__ int wave_largest[kBlock / kWave];
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) largest = max(largest, __shfl_xor(largest, d, kWave));
    if (threadIdx.x % kWave == 0) wave_largest[threadIdx.x / kWave] = largest;
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 1; w < kBlock / kWave; ++w) largest = max(largest, wave_largest[w]);
        if (largest > 0) atomicMax(summary + 1, largest);  // one per workgroup: integer maximum, any order
    }
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

struct GroupLayout {
    size_t col, counters, table, scan;
    size_t total() const { return 3 * col + counters + table + scan; }
};

}  // namespace

// The sort for the rest of the library (radix_sort.h).
size_t radix_sort_counter_bytes(int64_t N) { return radix_counter_bytes(N); }

int radix_sort_positions(const int32_t *keys, int64_t N, int bits, int32_t *keys_out, int32_t *pos_out,
                         int32_t *tmp_keys, int32_t *tmp_pos, void *counters, hipStream_t stream) {
    return radix_sort_by_key(keys, N, bits, keys_out, pos_out, tmp_keys, tmp_pos, counters, nullptr, 0, nullptr, nullptr,
                             stream);
}

size_t occupancy_scan_bytes(int64_t n);
int occupancy_scan(const int32_t *in, int64_t n, int32_t *out, void *scratch, hipStream_t stream);

namespace {

GroupLayout group_layout(int64_t N, int bits) {
    GroupLayout L;
    L.col = align_up((size_t)N * sizeof(int32_t), 256);
    L.counters = radix_counter_bytes(N);
    L.table = bits <= kTableBits ? align_up(((size_t)1 << bits) * sizeof(int32_t), 256) : 0;
    L.scan = bits <= kTableBits ? 0 : L.col + occupancy_scan_bytes(N);  // run heads + scan scratch
    return L;
}

}  // namespace

}  // namespace cgnn

using namespace cgnn;

extern "C" size_t cgnn_lsh_group_workspace_bytes(int64_t N, int bits) {
    if (N <= 0 || N >= INT32_MAX || bits < 0 || bits > 30) return 0;
    // two columns (sorted codes; the keys or the payload between passes), the sort's counters,
    // and the code table (up to 16 bits) or the run heads and their scan (beyond)
    return group_layout(N, bits).total();
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
    const GroupLayout L = group_layout(N, bits);
    char *base = static_cast<char *>(workspace);
    int32_t *sorted_code = reinterpret_cast<int32_t *>(base);
    int32_t *tmp_keys = reinterpret_cast<int32_t *>(base + L.col);
    int32_t *tmp_vals = reinterpret_cast<int32_t *>(base + 2 * L.col);
    void *counters = base + 3 * L.col;
    char *rest = base + 3 * L.col + L.counters;
    int64_t blocks = ceil_div(N, kBlock);
    if (blocks > 8192) blocks = 8192;
    const int64_t capacity = std::min<int64_t>(N, (int64_t)1 << bits);
    int64_t cblocks = ceil_div(capacity + 1, kBlock);
    if (cblocks > 4096) cblocks = 4096;
    int rc;
    if (bits <= kTableBits) {
        const int codes = 1 << bits;
        int32_t *table = reinterpret_cast<int32_t *>(rest);
        // with two passes the last one writes the ids straight into sorted_id
        bool ranked = false;
        int32_t *sorted = radix_passes(bits) > 1 ? sorted_id : sorted_code;
        rc = radix_sort_by_key(raw_code, N, bits, sorted, perm, tmp_keys, tmp_vals, counters, table, codes - 1, summary,
                               &ranked, stream);
        if (rc != CGNN_OK) return rc;
        int64_t fblocks = ceil_div(N, 4 * kBlock);  // four positions a thread
        if (fblocks > 8192) fblocks = 8192;
        hipLaunchKernelGGL(group_table_finish_kernel, dim3((unsigned)fblocks), dim3(kBlock), 0, stream, N, raw_code, sorted,
                           table, codes - 1, ranked, ids, sorted_id, offsets);
    } else {
        int32_t *head = reinterpret_cast<int32_t *>(rest);
        void *scan_scratch = rest + L.col;
        rc = radix_sort_by_key(raw_code, N, bits, sorted_code, perm, tmp_keys, tmp_vals, counters, nullptr, 0, nullptr,
                               nullptr, stream);
        if (rc != CGNN_OK) return rc;
        hipLaunchKernelGGL(group_heads_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, stream, sorted_code, N, head,
                           summary);
        rc = occupancy_scan(head, N, sorted_id, scan_scratch, stream);
        if (rc != CGNN_OK) return rc;
        hipLaunchKernelGGL(group_finish_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, stream, N, sorted_id, head,
                           perm, ids, offsets, summary);
    }
    hipLaunchKernelGGL(group_counts_kernel, dim3((unsigned)cblocks), dim3(kBlock), 0, stream, offsets, summary,
                       counts, capacity);
    return check_launch("lsh_group");
}

extern "C" size_t cgnn_cluster_members_workspace_bytes(int64_t N, int64_t groups) {
    if (N <= 0 || groups <= 0 || N >= INT32_MAX) return 0;
    // the keys (ids narrowed and clamped), two columns between passes, the sort's counters
    return 3 * align_up((size_t)N * sizeof(int32_t), 256) + radix_counter_bytes(N);
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
        if (workspace == nullptr || workspace_bytes < cgnn_cluster_members_workspace_bytes(N, groups))
            return fail(CGNN_EWORKSPACE, "cgnn_cluster_members: workspace too small");
        const size_t col = align_up((size_t)N * sizeof(int32_t), 256);
        char *base = static_cast<char *>(workspace);
        int32_t *keys = reinterpret_cast<int32_t *>(base);
        int32_t *tmp_keys = reinterpret_cast<int32_t *>(base + col);
        int32_t *tmp_vals = reinterpret_cast<int32_t *>(base + 2 * col);
        int64_t blocks = ceil_div(N, kBlock);
        if (blocks > 8192) blocks = 8192;
        hipLaunchKernelGGL(members_keys_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, stream, ids, keys, N, groups,
                           bad_id);
        int rc = radix_sort_by_key(keys, N, key_bits(groups), sorted_id, perm, tmp_keys, tmp_vals, base + 3 * col,
                                   nullptr, 0, nullptr, nullptr, stream);
        if (rc != CGNN_OK) return rc;
    }
    hipLaunchKernelGGL(members_offsets_kernel, dim3((unsigned)oblocks), dim3(kBlock), 0, stream,
                       sorted_id, N, offsets, groups);
    return check_launch("cluster_members");
}
