/*
 * CPU oracle of the neighbour sampler over a compressed graph: a plain-C restatement of
 * src/sample/csrc/neighbor_sample.h:27-131 (neighbor_sample_sim_impl), :134-211
 * (neighbor_sample_ori_impl) and src/sample/csrc/storage_api.h:6-118 (get_neighbor,
 * get_neighbor_list) of the reference (ZhengChenCS/CompressGNN).
 *
 * TEST INFRASTRUCTURE ONLY.  Only tests/ may load this; the product never does.
 *
 * The reference draws its random indices one at a time from torch's global CPU generator
 * (neighbor_sample.h:10-15).  Here the draws come from a callback, so that a test can hand in
 * that very generator (the sampling loop then reproduces the compiled reference exactly,
 * which is how this file is pinned: tests/test_oracle_sample.py against oracle/_ref and the
 * golden vectors written from it), or from the counter-based generator the HIP sampler uses
 * (oracle_counter_draw below: PARITY UNPINNED -- it is this build's own definition; the
 * reference has no device sampler, so the stream of random numbers on the GPU has nothing to
 * be compared with; what is compared is everything that follows from a given stream).
 * Further pins: the expansion invariant (the neighbours enumerated by get_neighbor over all
 * indices, and the full list, are the expanded in-list of the vertex) on graphs whose rule
 * hierarchy the reference's degree computation covers.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef struct {
    const int64_t *v2v_ptr, *v2v_idx, *v2r_ptr, *v2r_idx, *r2v_ptr, *r2v_idx;
    int levels;
    const int64_t *const *r2r_ptr;
    const int64_t *const *r2r_idx;
    const int64_t *v_degree, *r_degree;
} sample_graph;

/* storage_api.h:6-70.  Returns -1 where the reference throws std::out_of_range. */
static int64_t get_neighbor(const sample_graph *g, int64_t node, int64_t k) {
    const int64_t v2v_start = g->v2v_ptr[node], v2v_count = g->v2v_ptr[node + 1] - v2v_start;
    if (k < v2v_count) return g->v2v_idx[v2v_start + k];
    k -= v2v_count;
    const int64_t v2r_start = g->v2r_ptr[node], v2r_count = g->v2r_ptr[node + 1] - v2r_start;
    for (int64_t i = 0; i < v2r_count; ++i) {
        int64_t rule = g->v2r_idx[v2r_start + i];
        const int64_t degree = g->r_degree[rule];
        if (k < degree) {
            int layer = 0;
            while (layer < g->levels) {
                const int64_t s = g->r2v_ptr[rule], c = g->r2v_ptr[rule + 1] - s;
                if (k < c) return g->r2v_idx[s + k];
                k -= c;
                const int64_t rs = g->r2r_ptr[layer][rule], rc = g->r2r_ptr[layer][rule + 1] - rs;
                for (int64_t r = 0; r < rc; ++r) {
                    const int64_t child = g->r2r_idx[layer][rs + r];
                    const int64_t cd = g->r_degree[child];
                    if (k < cd) {
                        rule = child;
                        break;
                    }
                    k -= cd;
                }
                layer++;
            }
            const int64_t s = g->r2v_ptr[rule], c = g->r2v_ptr[rule + 1] - s;
            if (k < c) return g->r2v_idx[s + k];
            /* The descent found fewer entries than r_degree promised (degrees that do not fit the
             * hierarchy).  storage_api.h:57-64 goes on to the next rule with k - degree < 0 and
             * indexes before that rule's list (undefined behaviour); when no rule follows it throws
             * out_of_range.  Here both cases report out of range. */
            return -1;
        }
        k -= degree;
    }
    return -1;
}

typedef struct {
    int64_t *data;
    int64_t size, cap;
} vec64;

static void push(vec64 *v, int64_t x) {
    if (v->size == v->cap) {
        v->cap = v->cap ? 2 * v->cap : 64;
        v->data = (int64_t *)realloc(v->data, sizeof(int64_t) * (size_t)v->cap);
    }
    v->data[v->size++] = x;
}

/* storage_api.h:72-118: v2v entries, then the r2v entries of the rules reached from the
 * vertex, the rules in breadth-first order (level k of r2r expands the k-th wave). */
static void get_neighbor_list(const sample_graph *g, int64_t node, vec64 *out) {
    out->size = 0;
    for (int64_t e = g->v2v_ptr[node]; e < g->v2v_ptr[node + 1]; ++e) push(out, g->v2v_idx[e]);
    vec64 rules = {0, 0, 0};
    for (int64_t e = g->v2r_ptr[node]; e < g->v2r_ptr[node + 1]; ++e) push(&rules, g->v2r_idx[e]);
    int64_t begin = 0, end = rules.size;
    for (int k = 0; k < g->levels; ++k) {
        for (int64_t i = begin; i < end; ++i) {
            const int64_t rule = rules.data[i];
            for (int64_t e = g->r2r_ptr[k][rule]; e < g->r2r_ptr[k][rule + 1]; ++e) push(&rules, g->r2r_idx[k][e]);
        }
        begin = end;
        end = rules.size;
    }
    for (int64_t i = 0; i < rules.size; ++i) {
        const int64_t rule = rules.data[i];
        for (int64_t e = g->r2v_ptr[rule]; e < g->r2v_ptr[rule + 1]; ++e) push(out, g->r2v_idx[e]);
    }
    free(rules.data);
}

/* The counter-based generator of the HIP sampler (this build's definition): a draw depends on
 * (seed, layer, position of the frontier node among the samples, j) only. */
static uint64_t mix64(uint64_t z) {
    z ^= z >> 30;
    z *= 0xbf58476d1ce4e5b9ULL;
    z ^= z >> 27;
    z *= 0x94d049bb133111ebULL;
    z ^= z >> 31;
    return z;
}

int64_t oracle_counter_draw(uint64_t seed, int64_t layer, int64_t i, int64_t j, int64_t high) {
    const uint64_t key = mix64(seed ^ (0x9e3779b97f4a7c15ULL * (uint64_t)(layer + 1)));
    const uint64_t u = mix64(key + (uint64_t)i * 0xd1342543de82ef95ULL + (uint64_t)j);
    return (int64_t)(((unsigned __int128)u * (uint64_t)high) >> 64);
}

/* draw(high, layer, i, j, user) -> an integer in [0, high) */
typedef int64_t (*draw_fn)(int64_t high, int64_t layer, int64_t i, int64_t j, void *user);

static int64_t counter_draw_adapter(int64_t high, int64_t layer, int64_t i, int64_t j, void *user) {
    return oracle_counter_draw(*(const uint64_t *)user, layer, i, j, high);
}

/* neighbor_sample.h:27-131.  plain != 0: neighbor_sample_ori_impl (:134-211), where the graph
 * is (colptr, row) in v2v_ptr / v2v_idx and the roles of rows and cols are exchanged.
 * Results are returned in malloc'ed arrays the caller releases with oracle_free.  Return
 * value: 0, or -1 where the reference throws out_of_range. */
int oracle_neighbor_sample(int64_t vertex_cnt, const int64_t *v2v_ptr, const int64_t *v2v_idx, const int64_t *v2r_ptr,
                           const int64_t *v2r_idx, const int64_t *r2v_ptr, const int64_t *r2v_idx, int levels,
                           const int64_t *const *r2r_ptr, const int64_t *const *r2r_idx, const int64_t *v_degree,
                           const int64_t *r_degree, const int64_t *input, int64_t n_input, const int64_t *num_neighbors,
                           int n_layers, int plain, draw_fn draw, void *user, uint64_t counter_seed,
                           int64_t **samples_out, int64_t *n_samples, int64_t **rows_out, int64_t **cols_out,
                           int64_t *n_edges) {
    sample_graph g = {v2v_ptr, v2v_idx, v2r_ptr, v2r_idx, r2v_ptr, r2v_idx, levels, r2r_ptr, r2r_idx, v_degree, r_degree};
    if (draw == NULL) {
        draw = counter_draw_adapter;
        user = &counter_seed;
    }
    vec64 samples = {0, 0, 0}, rows = {0, 0, 0}, cols = {0, 0, 0}, list = {0, 0, 0}, chosen = {0, 0, 0};
    int64_t *local = (int64_t *)malloc(sizeof(int64_t) * (size_t)(vertex_cnt > 0 ? vertex_cnt : 1));
    for (int64_t v = 0; v < vertex_cnt; ++v) local[v] = -1;
    for (int64_t i = 0; i < n_input; ++i) {
        push(&samples, input[i]);
        if (local[input[i]] < 0) local[input[i]] = i;
    }
    int status = 0;
    int64_t begin = 0, end = samples.size;
    for (int ell = 0; ell < n_layers && status == 0; ++ell) {
        const int64_t num_samples = num_neighbors[ell];
        for (int64_t i = begin; i < end && status == 0; ++i) {
            const int64_t w = samples.data[i];
            const int64_t degree = plain ? v2v_ptr[w + 1] - v2v_ptr[w] : v_degree[w];
            if (degree == 0) continue;
            list.size = 0;
            if (num_samples >= degree) {
                if (plain)
                    for (int64_t e = v2v_ptr[w]; e < v2v_ptr[w + 1]; ++e) push(&list, v2v_idx[e]);
                else
                    get_neighbor_list(&g, w, &list);
            } else {
                chosen.size = 0;
                for (int64_t j = degree - num_samples; j < degree; ++j) {
                    int64_t rnd = draw(j, ell, i, j, user);
                    int taken = 0;
                    for (int64_t c = 0; c < chosen.size; ++c) taken |= chosen.data[c] == rnd;
                    if (taken) rnd = j;
                    push(&chosen, rnd);
                    const int64_t nb = plain ? v2v_idx[v2v_ptr[w] + rnd] : get_neighbor(&g, w, rnd);
                    if (nb < 0) {
                        status = -1;
                        break;
                    }
                    push(&list, nb);
                }
            }
            for (int64_t t = 0; t < list.size && status == 0; ++t) {
                const int64_t nb = list.data[t];
                if (local[nb] < 0) {
                    local[nb] = samples.size;
                    push(&samples, nb);
                }
                push(plain ? &cols : &rows, i);
                push(plain ? &rows : &cols, local[nb]);
            }
        }
        begin = end;
        end = samples.size;
    }
    free(local);
    free(list.data);
    free(chosen.data);
    *samples_out = samples.data;
    *n_samples = samples.size;
    *rows_out = rows.data;
    *cols_out = cols.data;
    *n_edges = rows.size;
    return status;
}

/* get_neighbor for a list of (node, index) pairs; -1 where the reference throws. */
void oracle_get_neighbors(const int64_t *v2v_ptr, const int64_t *v2v_idx, const int64_t *v2r_ptr, const int64_t *v2r_idx,
                          const int64_t *r2v_ptr, const int64_t *r2v_idx, int levels, const int64_t *const *r2r_ptr,
                          const int64_t *const *r2r_idx, const int64_t *v_degree, const int64_t *r_degree, int64_t n,
                          const int64_t *nodes, const int64_t *indices, int64_t *out) {
    sample_graph g = {v2v_ptr, v2v_idx, v2r_ptr, v2r_idx, r2v_ptr, r2v_idx, levels, r2r_ptr, r2r_idx, v_degree, r_degree};
    for (int64_t t = 0; t < n; ++t) out[t] = get_neighbor(&g, nodes[t], indices[t]);
}

/* get_neighbor_list of one vertex; the list is malloc'ed (oracle_free). */
int64_t oracle_neighbor_list(const int64_t *v2v_ptr, const int64_t *v2v_idx, const int64_t *v2r_ptr, const int64_t *v2r_idx,
                             const int64_t *r2v_ptr, const int64_t *r2v_idx, int levels, const int64_t *const *r2r_ptr,
                             const int64_t *const *r2r_idx, int64_t node, int64_t **out) {
    sample_graph g = {v2v_ptr, v2v_idx, v2r_ptr, v2r_idx, r2v_ptr, r2v_idx, levels, r2r_ptr, r2r_idx, NULL, NULL};
    vec64 list = {0, 0, 0};
    get_neighbor_list(&g, node, &list);
    *out = list.data;
    return list.size;
}

void oracle_free(void *p) { free(p); }
