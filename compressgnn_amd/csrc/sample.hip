// Neighbour sampling over a compressed graph on the device: the work of the reference's CPU
// module compressgnn_sample (src/sample/csrc/neighbor_sample.h:27-131 with
// src/sample/csrc/storage_api.h:6-118; the plain-CSC form :134-211 is the case without rules).
//
// One layer of sampling is four steps, each an entry point here:
//   count    a wave per frontier vertex: how many neighbours the vertex contributes (all of
//            them when the fan-out covers its degree, else the fan-out);
//   (prefix sums of the counts: cgnn_exclusive_sum_i32)
//   fill     a wave per frontier vertex writes its neighbours: the whole expanded in-list in the
//            reference's order (v2v entries, then the r2v entries of the rules reached from the
//            vertex in breadth-first order), or the neighbours at `fan-out` distinct random
//            positions of the expanded list (the reference's selection loop, with positions
//            resolved by descending through the rule levels with the expanded degrees);
//   relabel  local numbers for the neighbours: a vertex seen before keeps its number, new ones
//            are numbered in the order of their first occurrence, as the reference's hash map
//            does; here with a table over all vertices, integer atomic minima and a prefix sum,
//            so the numbering does not depend on timing.
//
// The breadth-first order of the full list is produced without a queue: a depth-first walk
// visits the rules of one depth in the same left-to-right order as the breadth-first walk
// does, so a first walk adds up the r2v sizes per depth and a second walk writes every rule's
// entries at (entries of shallower depths) + (entries of rules of its depth visited so far).
//
// Random positions come from a counter-based generator (a draw depends on the seed, the layer,
// the position of the frontier vertex among the samples and the step of the selection loop),
// so a sample does not depend on scheduling.  The reference draws from torch's sequential CPU
// generator; the streams differ by construction, everything downstream of a stream is the same.
#include "common.h"

namespace cgnn {

size_t occupancy_scan_bytes(int64_t n);
int occupancy_scan(const int32_t *in, int64_t n, int32_t *out, void *scratch, hipStream_t stream);

namespace {

constexpr int kUnseen = INT32_MAX;
constexpr int kLdsPicks = 1024;  // random positions a wave keeps in LDS

struct Graph {
    const int64_t *v2v_ptr, *v2v_idx, *v2r_ptr, *v2r_idx, *r2v_ptr, *r2v_idx;
    const int64_t *r2r_ptr[CGNN_SAMPLE_MAX_LEVELS], *r2r_idx[CGNN_SAMPLE_MAX_LEVELS];
    const int64_t *v_degree, *r_degree;
    int64_t vertex_cnt, rule_cnt;
    int levels;
};

Graph graph_of(const cgnn_sample_graph *g) {
    Graph d{};
    d.v2v_ptr = g->v2v_ptr, d.v2v_idx = g->v2v_idx, d.v2r_ptr = g->v2r_ptr, d.v2r_idx = g->v2r_idx;
    d.r2v_ptr = g->r2v_ptr, d.r2v_idx = g->r2v_idx;
    for (int k = 0; k < g->levels; ++k) d.r2r_ptr[k] = g->r2r_ptr[k], d.r2r_idx[k] = g->r2r_idx[k];
    d.v_degree = g->v_degree, d.r_degree = g->r_degree;
    d.vertex_cnt = g->vertex_cnt, d.rule_cnt = g->rule_cnt, d.levels = g->levels;
    return d;
}

// ---------------------------------------------------------------- random positions --
__device__ __forceinline__ uint64_t mix64(uint64_t z) {
    z ^= z >> 30;
    z *= 0xbf58476d1ce4e5b9ULL;
    z ^= z >> 27;
    z *= 0x94d049bb133111ebULL;
    z ^= z >> 31;
    return z;
}

// an integer in [0, high)
__device__ __forceinline__ int64_t draw(uint64_t seed, int64_t layer, int64_t i, int64_t j, int64_t high) {
    const uint64_t key = mix64(seed ^ (0x9e3779b97f4a7c15ULL * (uint64_t)(layer + 1)));
    const uint64_t u = mix64(key + (uint64_t)i * 0xd1342543de82ef95ULL + (uint64_t)j);
    return (int64_t)__umul64hi(u, (uint64_t)high);
}

// -------------------------------------------------------- the expanded in-list ------
// The k-th neighbour in the order of storage_api.h:6-70: v2v entries; then, rule by rule of
// the vertex's v2r entries, the rule's expanded list (its r2v entries, then its children's
// lists, the children of the wave-th descent taken from level `wave` of r2r).  -1: k lies
// beyond what the descent finds (the reference throws out_of_range, or reads out of bounds: below).
__device__ int64_t neighbor_at(const Graph &g, int64_t node, int64_t k) {
    const int64_t v2v_start = g.v2v_ptr[node], v2v_count = g.v2v_ptr[node + 1] - v2v_start;
    if (k < v2v_count) return g.v2v_idx[v2v_start + k];
    if (g.v2r_ptr == nullptr) return -1;  // a plain graph: no rules
    k -= v2v_count;
    for (int64_t e = g.v2r_ptr[node]; e < g.v2r_ptr[node + 1]; ++e) {
        int64_t rule = g.v2r_idx[e];
        const int64_t degree = g.r_degree[rule];
        if (k < degree) {
            for (int level = 0; level < g.levels; ++level) {
                const int64_t own = g.r2v_ptr[rule], own_count = g.r2v_ptr[rule + 1] - own;
                if (k < own_count) return g.r2v_idx[own + k];
                k -= own_count;
                for (int64_t c = g.r2r_ptr[level][rule]; c < g.r2r_ptr[level][rule + 1]; ++c) {
                    const int64_t child = g.r2r_idx[level][c];
                    const int64_t child_degree = g.r_degree[child];
                    if (k < child_degree) {
                        rule = child;
                        break;
                    }
                    k -= child_degree;
                }
            }
            const int64_t own = g.r2v_ptr[rule], own_count = g.r2v_ptr[rule + 1] - own;
            if (k < own_count) return g.r2v_idx[own + k];
            // The descent found less than r_degree promised (degrees that do not fit the hierarchy).
            // The reference goes on to the next rule with k - degree, which is negative by now, and
            // indexes before that rule's list; here the position counts as out of range.
            return -1;
        }
        k -= degree;
    }
    return -1;
}

// Depth-first walk over the rules reached from `node` (depth d expands through level d of
// r2r; rules at depth `levels` are not expanded): visit(rule, depth) in pre-order.  The walk is
// uniform over the wave (every lane runs it on the same vertex).
template <typename Visit>
__device__ __forceinline__ void walk_rules(const Graph &g, int64_t node, Visit visit) {
    int64_t at[CGNN_SAMPLE_MAX_LEVELS + 1], end[CGNN_SAMPLE_MAX_LEVELS + 1];
    if (g.v2r_ptr == nullptr) return;  // a plain graph: no rules
    for (int64_t e = g.v2r_ptr[node]; e < g.v2r_ptr[node + 1]; ++e) {
        int64_t rule = g.v2r_idx[e];
        int depth = 0;
        visit(rule, 0);
        if (g.levels > 0) {
            at[0] = g.r2r_ptr[0][rule];
            end[0] = g.r2r_ptr[0][rule + 1];
        }
        // the stack holds, per depth, the range of children still to visit
        while (g.levels > 0 && depth >= 0) {
            if (at[depth] == end[depth]) {
                --depth;
                continue;
            }
            rule = g.r2r_idx[depth][at[depth]++];
            visit(rule, depth + 1);
            if (depth + 1 < g.levels) {
                ++depth;
                at[depth] = g.r2r_ptr[depth][rule];
                end[depth] = g.r2r_ptr[depth][rule + 1];
            }
        }
    }
}

// Length of the full list of storage_api.h:72-118 and the r2v entries per depth.
__device__ int64_t full_list_sizes(const Graph &g, int64_t node, int64_t per_depth[CGNN_SAMPLE_MAX_LEVELS + 1]) {
    for (int d = 0; d <= g.levels; ++d) per_depth[d] = 0;
    walk_rules(g, node, [&](int64_t rule, int depth) { per_depth[depth] += g.r2v_ptr[rule + 1] - g.r2v_ptr[rule]; });
    int64_t total = g.v2v_ptr[node + 1] - g.v2v_ptr[node];
    for (int d = 0; d <= g.levels; ++d) total += per_depth[d];
    return total;
}

struct LayerArgs {
    Graph g;
    const int64_t *frontier;  // [n] vertices
    int64_t n;
    int64_t fanout;
    int64_t first_position;   // position of frontier[0] among the samples
    int64_t layer;
    uint64_t seed;
    int32_t *counts;          // [n]
    const int32_t *offsets;   // [n + 1]
    int64_t *neighbors;       // [offsets[n]]
    int64_t *sources;         // [offsets[n]] position (among the samples) of the vertex a neighbour belongs to
    int64_t *picks;           // [offsets[n]] scratch: the chosen positions
    int32_t *status;          // device flags, see CGNN_SAMPLE_* in the header
};

__device__ __forceinline__ int64_t degree_of(const Graph &g, int64_t node) {
    return g.v_degree ? g.v_degree[node] : g.v2v_ptr[node + 1] - g.v2v_ptr[node];
}

// counts[i]: neighbours that frontier vertex i contributes (neighbor_sample.h:88-99,111).
__global__ __launch_bounds__(kBlock) void sample_count_kernel(LayerArgs a) {
    const int64_t i = (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
    if (i >= a.n) return;
    const int64_t node = a.frontier[i];
    int32_t count = 0;
    if (node < 0 || node >= a.g.vertex_cnt) {
        *a.status = CGNN_SAMPLE_BAD_VERTEX;  // every writer of a kind stores the same value
    } else {
        const int64_t degree = degree_of(a.g, node);
        if (degree > 0) {
            if (a.fanout >= degree) {
                int64_t per_depth[CGNN_SAMPLE_MAX_LEVELS + 1];
                const int64_t full = full_list_sizes(a.g, node, per_depth);
                if (full >= INT32_MAX) *a.status = CGNN_SAMPLE_TOO_MANY;
                else count = (int32_t)full;
            } else if (a.fanout >= INT32_MAX) {
                *a.status = CGNN_SAMPLE_TOO_MANY;  // one vertex alone would add 2^31 - 1 neighbours or more
            } else {
                count = (int32_t)a.fanout;
            }
        }
    }
    if (threadIdx.x % kWave == 0) a.counts[i] = count;
}

__global__ __launch_bounds__(kBlock) void sample_fill_kernel(LayerArgs a) {
    const int lane = threadIdx.x % kWave;
    const int64_t i = (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
    if (i >= a.n) return;
    const int64_t out0 = a.offsets[i], count = a.offsets[i + 1] - out0;
    if (count == 0) return;
    const Graph &g = a.g;
    const int64_t node = a.frontier[i];  // in range: the count of a vertex out of range is 0
    const int64_t position = a.first_position + i;
    for (int64_t t = lane; t < count; t += kWave) a.sources[out0 + t] = position;
    const int64_t degree = degree_of(g, node);
    auto put = [&](int64_t slot, int64_t neighbor) {
        if (neighbor < 0 || neighbor >= g.vertex_cnt) {
            // -1: the descent ran out (out_of_range in the reference); anything else: a corrupt graph
            *a.status = neighbor == -1 ? CGNN_SAMPLE_OUT_OF_RANGE : CGNN_SAMPLE_BAD_VERTEX;
            neighbor = 0;
        }
        a.neighbors[out0 + slot] = neighbor;
    };
    if (a.fanout >= degree) {
        // the whole list: v2v entries, then per depth the r2v entries of the rules of that depth
        const int64_t v2v_start = g.v2v_ptr[node], v2v_count = g.v2v_ptr[node + 1] - v2v_start;
        for (int64_t t = lane; t < v2v_count; t += kWave) put(t, g.v2v_idx[v2v_start + t]);
        int64_t next[CGNN_SAMPLE_MAX_LEVELS + 1];  // where the next rule of a depth writes
        full_list_sizes(g, node, next);
        int64_t running = v2v_count;
        for (int d = 0; d <= g.levels; ++d) {
            const int64_t size = next[d];
            next[d] = running;
            running += size;
        }
        walk_rules(g, node, [&](int64_t rule, int depth) {
            const int64_t own = g.r2v_ptr[rule], own_count = g.r2v_ptr[rule + 1] - own;
            for (int64_t t = lane; t < own_count; t += kWave) put(next[depth] + t, g.r2v_idx[own + t]);
            next[depth] += own_count;
        });
        return;
    }
    // `count` = fanout distinct positions out of `degree` (neighbor_sample.h:112-118): step j draws
    // from [0, j) and takes j itself when the draw was taken before.  The steps depend on each
    // other, so the wave runs them one after the other; all lanes compare a draw with the
    // positions chosen so far, 64 at a time.  The positions are kept in LDS; a fan-out beyond
    // kLdsPicks keeps them in the caller's scratch, accessed around the vector cache (one
    // lane writes, all lanes read).
    __shared__ int64_t lds_picks[kBlock / kWave][kLdsPicks];
    int64_t *mine = lds_picks[threadIdx.x / kWave];
    int64_t *far = a.picks + out0;
    const bool in_lds = count <= kLdsPicks;
    auto pick_at = [&](int64_t c) {
        return in_lds ? mine[c] : __hip_atomic_load(far + c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };
    for (int64_t s = 0; s < count; ++s) {
        const int64_t j = degree - count + s;
        int64_t rnd = draw(a.seed, a.layer, position, j, j);
        bool taken = false;
        for (int64_t c0 = 0; c0 < s; c0 += kWave) {
            const int64_t c = c0 + lane;
            taken = taken || (__ballot(c < s && pick_at(c) == rnd) != 0);
        }
        if (taken) rnd = j;
        if (lane == 0) {
            if (in_lds) mine[s] = rnd;
            else __hip_atomic_store(far + s, rnd, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // the position is read by all lanes in the next step
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    for (int64_t t = lane; t < count; t += kWave) put(t, neighbor_at(g, node, pick_at(t)));
}

// ------------------------------------------------------------------- relabelling ----
// seen_at[v] = first position at which vertex v appears among the new neighbours (only for
// vertices without a local number yet).
__global__ void relabel_first_kernel(const int64_t *__restrict__ neighbors, int64_t total,
                                     const int32_t *__restrict__ local_of, int32_t *__restrict__ seen_at) {
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        const int64_t v = neighbors[t];
        if (local_of[v] == kUnseen) atomicMin(&seen_at[v], (int32_t)t);  // integer minimum: any order, one result
    }
}

// introduces[t] = 1 where position t is the first occurrence of a vertex without a number.
__global__ void relabel_flag_kernel(const int64_t *__restrict__ neighbors, int64_t total,
                                    const int32_t *__restrict__ local_of, const int32_t *__restrict__ seen_at,
                                    int32_t *__restrict__ introduces) {
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        const int64_t v = neighbors[t];
        introduces[t] = (local_of[v] == kUnseen && seen_at[v] == (int32_t)t) ? 1 : 0;
    }
}

// New vertices take the numbers base, base + 1, ... in the order of their first occurrence.
__global__ void relabel_assign_kernel(const int64_t *__restrict__ neighbors, int64_t total,
                                      const int32_t *__restrict__ introduces, const int32_t *__restrict__ rank,
                                      int64_t base, int32_t *__restrict__ local_of, int64_t *__restrict__ samples,
                                      int64_t *__restrict__ new_count) {
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        if (introduces[t]) {
            const int64_t v = neighbors[t];
            const int64_t number = base + rank[t] - 1;  // rank: inclusive count of introductions up to t
            local_of[v] = (int32_t)number;
            samples[number] = v;
        }
        if (t == total - 1) *new_count = rank[t];
    }
}

__global__ void relabel_lookup_kernel(const int64_t *__restrict__ neighbors, int64_t total,
                                      const int32_t *__restrict__ local_of, int32_t *__restrict__ seen_at,
                                      int64_t *__restrict__ numbers) {
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        const int64_t v = neighbors[t];
        numbers[t] = local_of[v];
        seen_at[v] = kUnseen;  // the table is clean again for the next layer
    }
}

// The input vertices number themselves 0, 1, ...; of equal ones the first counts.
__global__ void relabel_seeds_kernel(const int64_t *__restrict__ input, int64_t n, int64_t vertex_cnt,
                                     int32_t *__restrict__ local_of, int32_t *__restrict__ status) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t v = input[i];
        if (v < 0 || v >= vertex_cnt) *status = CGNN_SAMPLE_BAD_VERTEX;
        else atomicMin(&local_of[v], (int32_t)i);
    }
}

__global__ void fill_i32_value_kernel(int32_t *p, int64_t n, int32_t value) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        p[i] = value;
}

// ---------------------------------------------------------------- prefix sums -------
// out[0] = 0, out[i + 1] = in[0] + ... + in[i] (n + 1 entries), three passes over tiles.
constexpr int kSumItems = 16;
constexpr int kSumTile = kBlock * kSumItems;

__device__ __forceinline__ int64_t block_sum_scan(int64_t v, int64_t *total) {
    __shared__ int64_t wave_sum[kBlock / kWave];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    int64_t inc = v;
#pragma unroll
    for (int s = 1; s < kWave; s <<= 1) {
        const int64_t n = __shfl_up(inc, s, kWave);
        if (lane >= s) inc += n;
    }
    __syncthreads();
    if (lane == kWave - 1) wave_sum[wave] = inc;
    __syncthreads();
    int64_t before = 0, all = 0;
#pragma unroll
    for (int w = 0; w < kBlock / kWave; ++w) {
        if (w < wave) before += wave_sum[w];
        all += wave_sum[w];
    }
    *total = all;
    return before + inc;
}

__global__ __launch_bounds__(kBlock) void sum_tiles_kernel(const int32_t *__restrict__ in, int64_t n,
                                                          int64_t *__restrict__ tile_total) {
    const int64_t base = (int64_t)blockIdx.x * kSumTile + (int64_t)threadIdx.x * kSumItems;
    int64_t s = 0;
#pragma unroll
    for (int k = 0; k < kSumItems; ++k)
        if (base + k < n) s += in[base + k];
    int64_t total;
    block_sum_scan(s, &total);
    if (threadIdx.x == 0) tile_total[blockIdx.x] = total;
}

__global__ __launch_bounds__(kBlock) void sum_totals_kernel(int64_t *tile_total, int64_t tiles) {
    int64_t running = 0;
    for (int64_t base = 0; base < tiles; base += kBlock) {
        const int64_t i = base + threadIdx.x;
        const int64_t v = i < tiles ? tile_total[i] : 0;
        int64_t total;
        const int64_t inc = block_sum_scan(v, &total);
        if (i < tiles) tile_total[i] = running + inc - v;
        running += total;
    }
}

__global__ __launch_bounds__(kBlock) void sum_apply_kernel(const int32_t *__restrict__ in, int64_t n,
                                                          const int64_t *__restrict__ tile_total,
                                                          int32_t *__restrict__ out, int32_t *__restrict__ status) {
    const int64_t base = (int64_t)blockIdx.x * kSumTile + (int64_t)threadIdx.x * kSumItems;
    int32_t v[kSumItems];
    int64_t s = 0;
#pragma unroll
    for (int k = 0; k < kSumItems; ++k) {
        v[k] = base + k < n ? in[base + k] : 0;
        s += v[k];
    }
    int64_t total;
    int64_t run = tile_total[blockIdx.x] + block_sum_scan(s, &total) - s;
    if (blockIdx.x == 0 && threadIdx.x == 0) out[0] = 0;
#pragma unroll
    for (int k = 0; k < kSumItems; ++k) {
        run += v[k];
        if (base + k < n) {
            if (run >= INT32_MAX) {
                if (status) *status = CGNN_SAMPLE_TOO_MANY;
                out[base + k + 1] = INT32_MAX;
            } else {
                out[base + k + 1] = (int32_t)run;
            }
        }
    }
}

int check_graph(const cgnn_sample_graph *g, const char *name) {
    if (g == nullptr) return fail(CGNN_EINVAL, "sample: null graph");
    if (g->vertex_cnt < 0 || g->rule_cnt < 0 || g->vertex_cnt >= INT32_MAX) {
        set_error("%s: vertex_cnt must be in [0, 2^31 - 1) and rule_cnt non-negative", name);
        return CGNN_EINVAL;
    }
    if (g->levels < 0 || g->levels > CGNN_SAMPLE_MAX_LEVELS) {
        set_error("%s: %d rule levels, at most %d are supported", name, g->levels, CGNN_SAMPLE_MAX_LEVELS);
        return CGNN_EUNSUPPORTED;
    }
    bool ok = g->v2v_ptr != nullptr;
    if (g->rule_cnt > 0) ok = ok && g->v2r_ptr && g->r2v_ptr;  // a graph without rules may leave the rule blocks out
    if (g->rule_cnt == 0 && (g->v2r_ptr == nullptr) != (g->r2v_ptr == nullptr)) ok = false;
    for (int k = 0; k < g->levels; ++k) ok = ok && g->r2r_ptr[k];
    if (!ok) {
        set_error("%s: a row-pointer array of the graph is null", name);
        return CGNN_EINVAL;
    }
    if (g->rule_cnt > 0 && (g->v_degree == nullptr || g->r_degree == nullptr)) {
        set_error("%s: a graph with rules needs the expanded degrees", name);
        return CGNN_EINVAL;
    }
    return CGNN_OK;
}

LayerArgs layer_args(const cgnn_sample_graph *g, int64_t n, const int64_t *frontier, int64_t fanout, int32_t *status) {
    LayerArgs a{};
    a.g = graph_of(g);
    a.frontier = frontier;
    a.n = n;
    a.fanout = fanout;
    a.status = status;
    return a;
}

unsigned blocks_for(int64_t n) {
    int64_t b = ceil_div(n, kBlock);
    return (unsigned)(b > 16384 ? 16384 : (b < 1 ? 1 : b));
}

}  // namespace
}  // namespace cgnn

using namespace cgnn;

extern "C" size_t cgnn_exclusive_sum_workspace_bytes(int64_t n) {
    return align_up((size_t)ceil_div(n < 1 ? 1 : n, kSumTile) * sizeof(int64_t), 256);
}

extern "C" int cgnn_exclusive_sum_i32(int64_t n, const int32_t *in, int32_t *out, int32_t *status, void *workspace,
                                      size_t workspace_bytes, cgnn_stream_t stream) {
    CGNN_REQUIRE(n >= 0 && n < INT32_MAX, "cgnn_exclusive_sum_i32: n must be in [0, 2^31 - 1)");
    CGNN_REQUIRE(out != nullptr, "cgnn_exclusive_sum_i32: out is null");
    if (n == 0) {
        hipLaunchKernelGGL(fill_i32_value_kernel, dim3(1), dim3(1), 0, stream, out, (int64_t)1, 0);
        return check_launch("exclusive_sum");
    }
    CGNN_REQUIRE(in != nullptr, "cgnn_exclusive_sum_i32: in is null");
    if (workspace == nullptr || workspace_bytes < cgnn_exclusive_sum_workspace_bytes(n))
        return fail(CGNN_EWORKSPACE, "cgnn_exclusive_sum_i32: workspace too small");
    const int64_t tiles = ceil_div(n, kSumTile);
    int64_t *totals = static_cast<int64_t *>(workspace);
    hipLaunchKernelGGL(sum_tiles_kernel, dim3((unsigned)tiles), dim3(kBlock), 0, stream, in, n, totals);
    hipLaunchKernelGGL(sum_totals_kernel, dim3(1), dim3(kBlock), 0, stream, totals, tiles);
    hipLaunchKernelGGL(sum_apply_kernel, dim3((unsigned)tiles), dim3(kBlock), 0, stream, in, n, totals, out, status);
    return check_launch("exclusive_sum");
}

extern "C" int cgnn_sample_count(const cgnn_sample_graph *graph, int64_t n, const int64_t *frontier, int64_t fanout,
                                 int32_t *counts, int32_t *status, cgnn_stream_t stream) {
    int rc = check_graph(graph, "cgnn_sample_count");
    if (rc != CGNN_OK) return rc;
    CGNN_REQUIRE(n >= 0 && n < INT32_MAX, "cgnn_sample_count: n must be in [0, 2^31 - 1)");
    CGNN_REQUIRE(fanout >= 0, "cgnn_sample_count: the fan-out must not be negative");
    if (n == 0) return CGNN_OK;
    CGNN_REQUIRE(frontier && counts && status, "cgnn_sample_count: null array");
    LayerArgs a = layer_args(graph, n, frontier, fanout, status);
    a.counts = counts;
    hipLaunchKernelGGL(sample_count_kernel, dim3((unsigned)ceil_div(n, kBlock / kWave)), dim3(kBlock), 0, stream, a);
    return check_launch("sample_count");
}

extern "C" int cgnn_sample_fill(const cgnn_sample_graph *graph, int64_t n, const int64_t *frontier, int64_t fanout,
                                const int32_t *offsets, int64_t first_position, int64_t layer, uint64_t seed,
                                int64_t *neighbors, int64_t *sources, int64_t *picks, int32_t *status,
                                cgnn_stream_t stream) {
    int rc = check_graph(graph, "cgnn_sample_fill");
    if (rc != CGNN_OK) return rc;
    CGNN_REQUIRE(n >= 0 && n < INT32_MAX, "cgnn_sample_fill: n must be in [0, 2^31 - 1)");
    CGNN_REQUIRE(fanout >= 0, "cgnn_sample_fill: the fan-out must not be negative");
    if (n == 0) return CGNN_OK;
    CGNN_REQUIRE(frontier && offsets && neighbors && sources && picks && status, "cgnn_sample_fill: null array");
    LayerArgs a = layer_args(graph, n, frontier, fanout, status);
    a.offsets = offsets;
    a.first_position = first_position;
    a.layer = layer;
    a.seed = seed;
    a.neighbors = neighbors;
    a.sources = sources;
    a.picks = picks;
    hipLaunchKernelGGL(sample_fill_kernel, dim3((unsigned)ceil_div(n, kBlock / kWave)), dim3(kBlock), 0, stream, a);
    return check_launch("sample_fill");
}

extern "C" int cgnn_sample_relabel_begin(int64_t vertex_cnt, int64_t n_input, const int64_t *input, int32_t *local_of,
                                         int32_t *seen_at, int32_t *status, cgnn_stream_t stream) {
    CGNN_REQUIRE(vertex_cnt >= 0 && vertex_cnt < INT32_MAX && n_input >= 0 && n_input < INT32_MAX,
                 "cgnn_sample_relabel_begin: sizes must be in [0, 2^31 - 1)");
    CGNN_REQUIRE(status != nullptr, "cgnn_sample_relabel_begin: status is null");
    hipLaunchKernelGGL(fill_i32_value_kernel, dim3(1), dim3(1), 0, stream, status, (int64_t)1, 0);
    if (vertex_cnt > 0) {
        CGNN_REQUIRE(local_of && seen_at, "cgnn_sample_relabel_begin: null table");
        hipLaunchKernelGGL(fill_i32_value_kernel, dim3(blocks_for(vertex_cnt)), dim3(kBlock), 0, stream, local_of,
                           vertex_cnt, kUnseen);
        hipLaunchKernelGGL(fill_i32_value_kernel, dim3(blocks_for(vertex_cnt)), dim3(kBlock), 0, stream, seen_at,
                           vertex_cnt, kUnseen);
    }
    if (n_input > 0) {
        CGNN_REQUIRE(input != nullptr, "cgnn_sample_relabel_begin: input is null");
        hipLaunchKernelGGL(relabel_seeds_kernel, dim3(blocks_for(n_input)), dim3(kBlock), 0, stream, input, n_input,
                           vertex_cnt, local_of, status);
    }
    return check_launch("sample_relabel_begin");
}

extern "C" size_t cgnn_sample_relabel_workspace_bytes(int64_t total) {
    if (total <= 0) return 0;
    return 2 * align_up((size_t)total * sizeof(int32_t), 256) + occupancy_scan_bytes(total);
}

extern "C" int cgnn_sample_relabel(int64_t total, const int64_t *neighbors, int64_t base, int32_t *local_of,
                                   int32_t *seen_at, int64_t *samples, int64_t *numbers, int64_t *new_count,
                                   void *workspace, size_t workspace_bytes, cgnn_stream_t stream) {
    CGNN_REQUIRE(total >= 0 && total < INT32_MAX && base >= 0 && base + total < INT32_MAX,
                 "cgnn_sample_relabel: sizes must stay below 2^31 - 1");
    CGNN_REQUIRE(new_count != nullptr, "cgnn_sample_relabel: new_count is null");
    if (total == 0) {
        hipLaunchKernelGGL(fill_i32_value_kernel, dim3(1), dim3(1), 0, stream, reinterpret_cast<int32_t *>(new_count),
                           (int64_t)2, 0);
        return check_launch("sample_relabel");
    }
    CGNN_REQUIRE(neighbors && local_of && seen_at && samples && numbers, "cgnn_sample_relabel: null array");
    if (workspace == nullptr || workspace_bytes < cgnn_sample_relabel_workspace_bytes(total))
        return fail(CGNN_EWORKSPACE, "cgnn_sample_relabel: workspace too small");
    const size_t col = align_up((size_t)total * sizeof(int32_t), 256);
    char *wbase = static_cast<char *>(workspace);
    int32_t *introduces = reinterpret_cast<int32_t *>(wbase);
    int32_t *rank = reinterpret_cast<int32_t *>(wbase + col);
    void *scan_scratch = wbase + 2 * col;
    const unsigned blocks = blocks_for(total);
    hipLaunchKernelGGL(relabel_first_kernel, dim3(blocks), dim3(kBlock), 0, stream, neighbors, total, local_of, seen_at);
    hipLaunchKernelGGL(relabel_flag_kernel, dim3(blocks), dim3(kBlock), 0, stream, neighbors, total, local_of, seen_at,
                       introduces);
    int rc = occupancy_scan(introduces, total, rank, scan_scratch, stream);
    if (rc != CGNN_OK) return rc;
    hipLaunchKernelGGL(relabel_assign_kernel, dim3(blocks), dim3(kBlock), 0, stream, neighbors, total, introduces, rank,
                       base, local_of, samples, new_count);
    hipLaunchKernelGGL(relabel_lookup_kernel, dim3(blocks), dim3(kBlock), 0, stream, neighbors, total, local_of, seen_at,
                       numbers);
    return check_launch("sample_relabel");
}
