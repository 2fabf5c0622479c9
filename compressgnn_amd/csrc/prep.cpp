// Host-side graph preparation (C ABI in include/compressgnn_prep.h): self loops,
// normalisation weights, stable transposes, the CompressGraph block partition, rule
// levels, expanded degrees, rule filters, the batch pair-merging compressor and the
// seeded synthetic graph generators.  Plain C++17, no GPU code.
//
// The routines that restate reference behaviour cite the reference file they follow
// (ZhengChenCS/CompressGNN, paths relative to its root); their outputs are compared
// bit for bit with the reference's own routines in tests/.
#include "compressgnn_prep.h"

#include <algorithm>
#include <climits>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <deque>
#include <numeric>
#include <parallel/algorithm>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

namespace {

thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

using i64 = int64_t;
using Rows = std::vector<std::vector<i64>>;

}  // namespace

struct cgnn_arrays {
    struct Item {
        int type;
        std::vector<i64> a64;
        std::vector<float> f32;
        std::vector<int32_t> a32;
    };
    std::vector<Item> items;
    std::vector<i64> scalars;

    void add(std::vector<i64> &&v) {
        items.emplace_back();
        items.back().type = CGNN_ARR_I64;
        items.back().a64 = std::move(v);
    }
    void add(std::vector<float> &&v) {
        items.emplace_back();
        items.back().type = CGNN_ARR_F32;
        items.back().f32 = std::move(v);
    }
    void add(std::vector<int32_t> &&v) {
        items.emplace_back();
        items.back().type = CGNN_ARR_I32;
        items.back().a32 = std::move(v);
    }
};

extern "C" {

int cgnn_arrays_count(const cgnn_arrays *a) { return a ? (int)a->items.size() : 0; }
int cgnn_arrays_type(const cgnn_arrays *a, int i) { return a->items.at(i).type; }
int64_t cgnn_arrays_size(const cgnn_arrays *a, int i) {
    const auto &it = a->items.at(i);
    switch (it.type) {
        case CGNN_ARR_I64: return (i64)it.a64.size();
        case CGNN_ARR_F32: return (i64)it.f32.size();
        default: return (i64)it.a32.size();
    }
}
const void *cgnn_arrays_data(const cgnn_arrays *a, int i) {
    const auto &it = a->items.at(i);
    switch (it.type) {
        case CGNN_ARR_I64: return it.a64.data();
        case CGNN_ARR_F32: return it.f32.data();
        default: return it.a32.data();
    }
}
int64_t cgnn_arrays_scalar(const cgnn_arrays *a, int i) { return a->scalars.at(i); }
void cgnn_arrays_free(cgnn_arrays *a) { delete a; }
const char *cgnn_prep_last_error(void) { return g_error; }

}  // extern "C"

namespace {

// ----------------------------------------------------------------- basic passes --

// Reference: src/offline/csrc/add_self_loop.h:17-43.  Rows are sorted; v goes where it
// belongs unless the row already holds it.
cgnn_arrays *add_self_loop(i64 V, const i64 *vlist, const i64 *elist) {
    auto *out = new cgnn_arrays;
    std::vector<i64> nv(V + 1, 0), ne;
    ne.reserve((size_t)vlist[V] + V);
    for (i64 v = 0; v < V; ++v) {
        i64 e = vlist[v];
        const i64 end = vlist[v + 1];
        while (e < end && elist[e] < v) ne.push_back(elist[e++]);
        if (e == end || elist[e] != v) ne.push_back(v);
        while (e < end) ne.push_back(elist[e++]);
        nv[v + 1] = (i64)ne.size();
    }
    out->add(std::move(nv));
    out->add(std::move(ne));
    return out;
}

// Stable counting sort by column.
cgnn_arrays *transpose(i64 rows, i64 cols, const i64 *vlist, const i64 *elist, const float *value) {
    const i64 nnz = vlist[rows];
    std::vector<i64> colptr(cols + 1, 0), row(nnz);
    std::vector<float> val(value ? nnz : 0);
    for (i64 e = 0; e < nnz; ++e) {
        if (elist[e] < 0 || elist[e] >= cols) {
            set_error("csr_transpose: column %lld out of range [0,%lld)", (long long)elist[e], (long long)cols);
            return nullptr;
        }
        ++colptr[elist[e] + 1];
    }
    for (i64 c = 0; c < cols; ++c) colptr[c + 1] += colptr[c];
    std::vector<i64> cursor(colptr.begin(), colptr.end() - 1);
    for (i64 r = 0; r < rows; ++r)
        for (i64 e = vlist[r]; e < vlist[r + 1]; ++e) {
            const i64 p = cursor[elist[e]]++;
            row[p] = r;
            if (value) val[p] = value[e];
        }
    auto *out = new cgnn_arrays;
    out->add(std::move(colptr));
    out->add(std::move(row));
    out->add(std::move(val));
    return out;
}

// Reference: src/offline/csrc/partition.h:14-110.  In every row the vertex columns
// (< V) come first; the first column >= V starts the rule part, rebased by -V.
cgnn_arrays *hybird_partition(i64 total, const i64 *vlist, const i64 *elist, const float *value, i64 V) {
    struct Block {
        std::vector<i64> ptr{0}, col;
        std::vector<float> val;
    } blk[4];  // v2v, v2r, r2v, r2r
    for (i64 r = 0; r < total; ++r) {
        Block &to_vertex = blk[r < V ? 0 : 2];
        Block &to_rule = blk[r < V ? 1 : 3];
        i64 e = vlist[r];
        const i64 end = vlist[r + 1];
        for (; e < end && elist[e] < V; ++e) {
            to_vertex.col.push_back(elist[e]);
            to_vertex.val.push_back(value[e]);
        }
        for (; e < end; ++e) {
            to_rule.col.push_back(elist[e] - V);
            to_rule.val.push_back(value[e]);
        }
        to_vertex.ptr.push_back((i64)to_vertex.col.size());
        to_rule.ptr.push_back((i64)to_rule.col.size());
    }
    auto *out = new cgnn_arrays;
    for (auto &b : blk) {
        out->add(std::move(b.ptr));
        out->add(std::move(b.col));
        out->add(std::move(b.val));
    }
    return out;
}

// Reference: src/offline/csrc/partition.h:112-216.  order 0 = rule without rule
// entries in its row; repeated ascending sweeps give order s to every rule whose row
// entries are all ordered (entries ordered earlier in the same sweep count).  Level k
// keeps the rows of order k+1; every level carries R+1 row pointers.
cgnn_arrays *topo_partition(i64 R, const i64 *vlist, const i64 *elist, const float *value) {
    std::vector<int> order(R, -1);
    i64 left = R;
    for (i64 r = 0; r < R; ++r)
        if (vlist[r + 1] == vlist[r]) {
            order[r] = 0;
            --left;
        }
    int sweep = 1;
    while (left > 0) {
        i64 progressed = 0;
        for (i64 r = 0; r < R; ++r) {
            if (order[r] != -1) continue;
            bool ready = true;
            for (i64 e = vlist[r]; e < vlist[r + 1]; ++e)
                if (order[elist[e]] == -1) {
                    ready = false;
                    break;
                }
            if (ready) {
                order[r] = sweep;
                --left;
                ++progressed;
            }
        }
        if (progressed == 0) {
            set_error("topo_partition: the rule block has a cycle");
            return nullptr;
        }
        ++sweep;
    }
    const int levels = sweep - 1;
    std::vector<std::vector<i64>> ptr(levels), col(levels);
    std::vector<std::vector<float>> val(levels);
    for (int k = 0; k < levels; ++k) ptr[k].reserve(R + 1), ptr[k].push_back(0);
    for (i64 r = 0; r < R; ++r) {
        const int k = order[r] - 1;
        if (k >= 0)
            for (i64 e = vlist[r]; e < vlist[r + 1]; ++e) {
                col[k].push_back(elist[e]);
                val[k].push_back(value[e]);
            }
        for (int j = 0; j < levels; ++j) ptr[j].push_back((i64)col[j].size());
    }
    auto *out = new cgnn_arrays;
    for (int k = 0; k < levels; ++k) {
        out->add(std::move(ptr[k]));
        out->add(std::move(col[k]));
        out->add(std::move(val[k]));
    }
    out->scalars.push_back(levels);
    return out;
}

// ------------------------------------------------------------------ rule filters --

// The rows of the compressed graph while rules are being inlined.  A row lives in the
// input arrays until it changes; only the rows that refer to an inlined rule (and the
// rules themselves) are ever copied out, so a filter pass costs a scan of the input plus
// work in proportion to what it inlines.
class EditedRows {
  public:
    EditedRows(i64 n, const i64 *vlist, const i64 *elist) : vlist_(vlist), elist_(elist), slot_(n, -1) {}
    i64 size_of(i64 n) const { return slot_[n] < 0 ? vlist_[n + 1] - vlist_[n] : (i64)edited_[slot_[n]].size(); }
    std::vector<i64> &edit(i64 n) {
        if (slot_[n] < 0) {
            slot_[n] = (int32_t)edited_.size();
            edited_.emplace_back(elist_ + vlist_[n], elist_ + vlist_[n + 1]);
        }
        return edited_[slot_[n]];
    }
    template <typename F>
    void for_each(i64 n, F f) const {
        if (slot_[n] < 0)
            for (i64 e = vlist_[n]; e < vlist_[n + 1]; ++e) f(elist_[e]);
        else
            for (i64 c : edited_[slot_[n]]) f(c);
    }

  private:
    const i64 *vlist_, *elist_;
    std::vector<int32_t> slot_;
    std::deque<std::vector<i64>> edited_;  // a deque: rows handed out by edit() stay where they are
};

// For every rule, the rows that refer to it, in ascending row order (one entry per
// reference).  The referrers of vertices are not kept: no filter decision reads them.
Rows rule_referrers(i64 V, i64 R, const i64 *vlist, const i64 *elist) {
    Rows t(R);
    for (i64 v = 0; v < V + R; ++v)
        for (i64 e = vlist[v]; e < vlist[v + 1]; ++e)
            if (elist[e] >= V) t[elist[e] - V].push_back(v);
    return t;
}

// Splice rule `id` into every row that refers to it (children keep their order and
// take the place of the reference), and let its rule children refer to those rows instead.
// Reference: src/offline/csrc/filter.h:30-66 / depth_filter.h:16-38.  `on_parent` and
// `on_child` see the rows whose statistics the caller tracks.
template <typename FP, typename FC>
void inline_rule(i64 id, i64 V, EditedRows &g, Rows &gt, FP on_parent, FC on_child) {
    std::vector<i64> body;  // a copy: no reference into the container is held while rows are copied out
    g.for_each(id, [&](i64 c) { body.push_back(c); });
    const std::vector<i64> &referrers = gt[id - V];
    for (size_t i = 0; i < referrers.size(); ++i) {
        const i64 parent = referrers[i];
        std::vector<i64> &row = g.edit(parent);
        auto pos = row.erase(std::find(row.begin(), row.end(), id));
        row.insert(pos, body.begin(), body.end());
        on_parent(parent);
    }
    for (size_t i = 0; i < body.size(); ++i) {
        const i64 child = body[i];
        if (child < V) continue;
        std::vector<i64> &refs = gt[child - V];
        auto pos = refs.erase(std::find(refs.begin(), refs.end(), id));
        refs.insert(pos, referrers.begin(), referrers.end());
        on_child(child);
    }
}

// Dense renumbering of the surviving rules and re-emission of all rows.
// Reference: src/offline/csrc/util.h:108-119,143-164.
cgnn_arrays *emit_filtered(const EditedRows &g, const std::vector<char> &dropped, i64 V, i64 R) {
    std::vector<i64> new_id(R);
    i64 next = V;
    for (i64 r = 0; r < R; ++r) {
        new_id[r] = next;
        if (!dropped[r]) ++next;
    }
    // where every surviving row starts, then all cores copy rows (most of a filter pass on a
    // large graph is this copy)
    std::vector<i64> nv((size_t)next + 1, 0);
    for (i64 n = 0; n < V + R; ++n) {
        if (n >= V && dropped[n - V]) continue;
        const i64 k = n < V ? n : new_id[n - V];
        nv[k + 1] = nv[k] + g.size_of(n);
    }
    std::vector<i64> ne((size_t)nv[next]);
#pragma omp parallel for schedule(static)
    for (i64 n = 0; n < V + R; ++n) {
        if (n >= V && dropped[n - V]) continue;
        i64 at = nv[n < V ? n : new_id[n - V]];
        g.for_each(n, [&](i64 c) { ne[at++] = c >= V ? new_id[c - V] : c; });
    }
    auto *out = new cgnn_arrays;
    out->add(std::move(nv));
    out->add(std::move(ne));
    out->scalars.push_back(V);
    out->scalars.push_back(next - V);
    return out;
}

// Reference: src/offline/csrc/filter.h:26-28,68-118.
cgnn_arrays *filter_csr(i64 V, i64 R, const i64 *vlist, const i64 *elist, int threshold) {
    EditedRows g(V + R, vlist, elist);
    Rows gt = rule_referrers(V, R, vlist, elist);
    std::vector<int> len(R), freq(R);
    std::vector<char> drop(R);
    auto small_saving = [&](int l, int f) { return (f - 1) * (l - 1) - 1 <= threshold; };
    for (i64 r = 0; r < R; ++r) {
        freq[r] = (int)gt[r].size();
        len[r] = (int)g.size_of(r + V);
        drop[r] = small_saving(len[r], freq[r]);
    }
    for (i64 r = 0; r < R; ++r) {
        if (!drop[r]) continue;
        const i64 id = r + V;
        const int grow = (int)g.size_of(id) - 1;
        inline_rule(
            id, V, g, gt,
            [&](i64 parent) {
                if (parent >= V) {
                    len[parent - V] += grow;
                    drop[parent - V] = small_saving(len[parent - V], freq[parent - V]);
                }
            },
            [&](i64 child) {
                // the reference adds the whole new referrer count here (filter.h:59)
                freq[child - V] += (int)gt[child - V].size();
                drop[child - V] = small_saving(len[child - V], freq[child - V]);
            });
    }
    return emit_filtered(g, drop, V, R);
}

// Reference: src/offline/csrc/gen_mask.h:180-233.  Vertices have order 0; a rule gets
// order s once every reference to it has been visited, s = sweep in which the last one
// was.  Returns the orders and the number of sweeps.
int vertex_order_csr(i64 V, i64 R, const i64 *vlist, const i64 *elist, std::vector<int32_t> &order) {
    constexpr int32_t kUnset = 100000;
    order.assign(V + R, kUnset);
    std::vector<int> pending(R, 0);
    const i64 E = vlist[V + R];
    for (i64 e = 0; e < E; ++e)
        if (elist[e] >= V) ++pending[elist[e] - V];
    std::vector<i64> work, next;
    work.reserve(V);
    for (i64 v = 0; v < V; ++v) {
        order[v] = 0;
        work.push_back(v);
    }
    int step = 1;
    while (!work.empty()) {
        for (i64 src : work)
            for (i64 e = vlist[src]; e < vlist[src + 1]; ++e) {
                const i64 dst = elist[e];
                if (dst >= V && order[dst] == kUnset && --pending[dst - V] == 0) {
                    order[dst] = step;
                    next.push_back(dst);
                }
            }
        ++step;
        work.swap(next);
        next.clear();
    }
    return step - 1;
}

// Reference: src/offline/csrc/gen_mask.h:111-174.  Rules that no other rule refers to
// have order 0; a rule referred to by rules gets the sweep in which its last referring
// rule was visited; vertices get the last sweep.  Returns the number of sweeps + 1.
int vertex_order_csc(i64 V, i64 R, const i64 *vlist, const i64 *elist, std::vector<int32_t> &order) {
    constexpr int32_t kUnset = 100000;
    order.assign(V + R, kUnset);
    std::vector<int> pending(R, 0);
    for (i64 r = 0; r < R; ++r)
        for (i64 e = vlist[r + V]; e < vlist[r + V + 1]; ++e)
            if (elist[e] >= V) ++pending[elist[e] - V];
    std::vector<i64> work, next;
    for (i64 r = 0; r < R; ++r)
        if (pending[r] == 0) {
            order[r + V] = 0;
            work.push_back(r + V);
        }
    int step = 1;
    while (!work.empty()) {
        for (i64 src : work)
            for (i64 e = vlist[src]; e < vlist[src + 1]; ++e) {
                const i64 dst = elist[e];
                if (dst >= V && order[dst] == kUnset && --pending[dst - V] == 0) {
                    order[dst] = step;
                    next.push_back(dst);
                }
            }
        ++step;
        work.swap(next);
        next.clear();
    }
    for (i64 v = 0; v < V; ++v) order[v] = step - 1;
    return step;
}

// Reference: src/offline/csrc/depth_filter.h:40-116.
cgnn_arrays *depth_filter_csr(i64 V, i64 R, const i64 *vlist, const i64 *elist, int max_depth, int min_edge) {
    EditedRows g(V + R, vlist, elist);
    Rows gt = rule_referrers(V, R, vlist, elist);
    std::vector<int32_t> depth;
    int deepest = vertex_order_csr(V, R, vlist, elist, depth);
    std::vector<char> drop(R, 0);
    std::vector<i64> edges_at(deepest + 1, 0);
    auto recount = [&](int upto) {
        for (int d = 0; d <= upto; ++d) edges_at[d] = 0;
        for (i64 r = 0; r < R; ++r)
            if (!drop[r] && depth[r + V] <= deepest) edges_at[depth[r + V]] += g.size_of(r + V);
    };
    for (i64 r = 0; r < R; ++r)
        if (depth[r + V] > deepest) {
            set_error("depth_filter_csr: rule %lld is unreachable from the vertices", (long long)r);
            return nullptr;
        }
    recount(deepest);
    int d = deepest;
    while (d >= max_depth) {
        if (edges_at[d] >= min_edge) {
            --d;
            continue;
        }
        for (i64 r = 0; r < R; ++r)
            if (depth[r + V] == d) {
                inline_rule(r + V, V, g, gt, [](i64) {}, [](i64) {});
                drop[r] = 1;
            }
        --d;
        if (d >= 0) recount(d);
    }
    return emit_filtered(g, drop, V, R);
}

// --------------------------------------------------- batch pair-merging compressor --
//
// Every round counts the adjacent pairs (a, b) over all vertex rows, turns each pair
// seen at least min_frequency times into a new rule node with children [a, b], and
// rewrites the rows left to right, replacing non-overlapping occurrences.  A pair that
// ends up replaced fewer than twice (because overlapping pairs were taken first) is
// not turned into a rule.  New rules get ascending ids in (a, b) order, so children
// always have smaller ids than their rule, and the expansion of every vertex row,
// in order, is the original row.  Rule bodies have two children and are never
// rewritten; longer shared runs become nested rules over the rounds.
cgnn_arrays *compress_batch(i64 V, const i64 *vlist, const i64 *elist, int rounds, int min_frequency) {
    const i64 E = vlist[V];
    std::vector<int32_t> seq(elist, elist + E), next_seq;
    std::vector<i64> ptr(vlist, vlist + V + 1), next_ptr(V + 1);
    std::vector<int32_t> rule_children;  // two per rule
    i64 R = 0;
    std::vector<uint64_t> keys;
    auto key_of = [](int32_t a, int32_t b) { return ((uint64_t)(uint32_t)a << 32) | (uint32_t)b; };
    for (int round = 0; round < rounds; ++round) {
        keys.clear();
        keys.reserve(seq.size());
        for (i64 v = 0; v < V; ++v)
            for (i64 e = ptr[v]; e + 1 < ptr[v + 1]; ++e) keys.push_back(key_of(seq[e], seq[e + 1]));
        std::sort(keys.begin(), keys.end());
        std::unordered_map<uint64_t, int32_t> cand;  // pair -> candidate index (ascending key order)
        std::vector<uint64_t> cand_key;
        for (size_t i = 0; i < keys.size();) {
            size_t j = i;
            while (j < keys.size() && keys[j] == keys[i]) ++j;
            if ((i64)(j - i) >= min_frequency) {
                cand.emplace(keys[i], (int32_t)cand_key.size());
                cand_key.push_back(keys[i]);
            }
            i = j;
        }
        if (cand_key.empty()) break;
        // pass 1: greedy parse with all candidates, count realised uses
        std::vector<int32_t> uses(cand_key.size(), 0);
        for (i64 v = 0; v < V; ++v)
            for (i64 e = ptr[v]; e < ptr[v + 1];) {
                if (e + 1 < ptr[v + 1]) {
                    auto it = cand.find(key_of(seq[e], seq[e + 1]));
                    if (it != cand.end()) {
                        ++uses[it->second];
                        e += 2;
                        continue;
                    }
                }
                ++e;
            }
        // keep candidates used at least twice; ids ascend with the pair key
        std::vector<int32_t> rule_id(cand_key.size(), -1);
        i64 added = 0;
        for (size_t c = 0; c < cand_key.size(); ++c)
            if (uses[c] >= 2) {
                if (V + R + added >= (i64)INT32_MAX) {
                    set_error("compress_csr_batch: node ids exceed int32");
                    return nullptr;
                }
                rule_id[c] = (int32_t)(V + R + added);
                rule_children.push_back((int32_t)(cand_key[c] >> 32));
                rule_children.push_back((int32_t)(cand_key[c] & 0xffffffffu));
                ++added;
            }
        if (added == 0) break;
        // pass 2: greedy parse with the kept candidates only
        next_seq.clear();
        next_seq.reserve(seq.size());
        for (i64 v = 0; v < V; ++v) {
            next_ptr[v] = (i64)next_seq.size();
            for (i64 e = ptr[v]; e < ptr[v + 1];) {
                if (e + 1 < ptr[v + 1]) {
                    auto it = cand.find(key_of(seq[e], seq[e + 1]));
                    if (it != cand.end() && rule_id[it->second] >= 0) {
                        next_seq.push_back(rule_id[it->second]);
                        e += 2;
                        continue;
                    }
                }
                next_seq.push_back(seq[e]);
                ++e;
            }
        }
        next_ptr[V] = (i64)next_seq.size();
        seq.swap(next_seq);
        ptr.swap(next_ptr);
        R += added;
    }
    std::vector<int32_t> out_ptr(V + R + 1), out_col;
    out_col.reserve(seq.size() + rule_children.size());
    for (i64 v = 0; v <= V; ++v) out_ptr[v] = (int32_t)ptr[v];
    out_col.insert(out_col.end(), seq.begin(), seq.end());
    out_col.insert(out_col.end(), rule_children.begin(), rule_children.end());
    for (i64 r = 0; r < R; ++r) out_ptr[V + r + 1] = (int32_t)(ptr[V] + 2 * (r + 1));
    auto *out = new cgnn_arrays;
    out->add(std::move(out_ptr));
    out->add(std::move(out_col));
    out->scalars.push_back(V);
    out->scalars.push_back(R);
    return out;
}

// ------------------------------------------------------------- synthetic graphs --

struct Rng {  // xoshiro256** seeded by splitmix64
    uint64_t s[4];
    explicit Rng(uint64_t seed) {
        for (auto &x : s) {
            seed += 0x9e3779b97f4a7c15ull;
            uint64_t z = seed;
            z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
            z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
            x = z ^ (z >> 31);
        }
    }
    static uint64_t rotl(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }
    uint64_t next() {
        const uint64_t r = rotl(s[1] * 5, 7) * 9, t = s[1] << 17;
        s[2] ^= s[0];
        s[3] ^= s[1];
        s[1] ^= s[2];
        s[0] ^= s[3];
        s[2] ^= t;
        s[3] = rotl(s[3], 45);
        return r;
    }
    double uniform() { return (double)(next() >> 11) * (1.0 / 9007199254740992.0); }
    i64 below(i64 n) { return (i64)(uniform() * (double)n); }
    int poisson(double lambda) {  // Knuth; lambda is small here
        const double limit = std::exp(-lambda);
        double p = 1.0;
        int k = 0;
        do {
            ++k;
            p *= uniform();
        } while (p > limit);
        return k - 1;
    }
};

cgnn_arrays *finish_rows(Rows &rows) {
    std::vector<i64> vl{0}, el;
    for (auto &r : rows) {
        std::sort(r.begin(), r.end());
        r.erase(std::unique(r.begin(), r.end()), r.end());
        el.insert(el.end(), r.begin(), r.end());
        vl.push_back((i64)el.size());
    }
    auto *out = new cgnn_arrays;
    out->add(std::move(vl));
    out->add(std::move(el));
    return out;
}

cgnn_arrays *gen_chung_lu(i64 V, i64 target_edges, double exponent, uint64_t seed) {
    Rng rng(seed);
    std::vector<double> w(V);
    double sum = 0;
    for (i64 i = 0; i < V; ++i) {
        w[i] = std::pow((double)(i + 1), -1.0 / (exponent - 1.0));
        sum += w[i];
    }
    for (auto &x : w) x *= (double)target_edges / sum;
    const double S = (double)target_edges;
    Rows rows(V);
    for (i64 i = 0; i < V; ++i)
        for (i64 j = 0; j < V; ++j) {
            if (i == j) continue;
            const double p = w[i] * w[j] / S;
            if (rng.uniform() < p) rows[i].push_back(j);
        }
    return finish_rows(rows);
}

cgnn_arrays *gen_copy_model(i64 V, double avg_degree, double copy_prob, uint64_t seed) {
    Rng rng(seed);
    Rows rows(V);
    const double fresh = avg_degree * (1.0 - copy_prob);
    for (i64 t = 1; t < V; ++t) {
        auto &row = rows[t];
        const auto &proto = rows[rng.below(t)];
        for (i64 n : proto)
            if (rng.uniform() < copy_prob) row.push_back(n);
        int extra = rng.poisson(fresh);
        if (t < 64) extra = (int)std::min<i64>(t, (i64)std::ceil(avg_degree));  // seed region: dense start
        for (int k = 0; k < extra; ++k) row.push_back(rng.below(t));
        std::sort(row.begin(), row.end());
        row.erase(std::unique(row.begin(), row.end()), row.end());
    }
    return finish_rows(rows);
}

template <typename F>
cgnn_arrays *guarded(F f) {
    try {
        return f();
    } catch (const std::exception &e) {
        set_error("%s", e.what());
        return nullptr;
    }
}

}  // namespace

extern "C" {

cgnn_arrays *cgnn_add_self_loop_csr(int64_t V, const int64_t *vlist, const int64_t *elist) {
    if (V < 0 || !vlist) {
        set_error("add_self_loop_csr: bad arguments");
        return nullptr;
    }
    return guarded([&] { return add_self_loop(V, vlist, elist); });
}

int cgnn_get_norm_degree(int64_t E, const int64_t *dst, int64_t V, float *out) {
    // Reference: src/offline/csrc/norm.h:20-45 -- the count is accumulated in float32
    // on top of 1e-6, then 1/sqrt in float32.
    if (E < 0 || V < 0 || (E > 0 && !dst) || (V > 0 && !out)) {
        set_error("get_norm_degree: bad arguments");
        return 1;
    }
    for (i64 v = 0; v < V; ++v) out[v] = (float)1e-6;
    for (i64 e = 0; e < E; ++e) {
        if (dst[e] < 0 || dst[e] >= V) {
            set_error("get_norm_degree: vertex %lld out of range", (long long)dst[e]);
            return 1;
        }
        out[dst[e]] += 1;
    }
    for (i64 v = 0; v < V; ++v) out[v] = 1 / std::sqrt(out[v]);
    return 0;
}

int cgnn_gcn_norm_csr_compress(int64_t V, int64_t R, const int64_t *vlist, const int64_t *elist,
                               const float *d, float *weight) {
    if (V < 0 || R < 0 || !vlist) {
        set_error("gcn_norm_csr_compress: bad arguments");
        return 1;
    }
    for (i64 n = 0; n < V + R; ++n)
        for (i64 e = vlist[n]; e < vlist[n + 1]; ++e) {
            const i64 c = elist[e];
            if (n < V) weight[e] = c < V ? d[n] * d[c] : d[n];
            else weight[e] = c < V ? d[c] : 1.0f;
        }
    return 0;
}

cgnn_arrays *cgnn_csr_transpose(int64_t rows, int64_t cols, const int64_t *vlist, const int64_t *elist,
                                const float *value) {
    if (rows < 0 || cols < 0 || !vlist) {
        set_error("csr_transpose: bad arguments");
        return nullptr;
    }
    return guarded([&] { return transpose(rows, cols, vlist, elist, value); });
}

cgnn_arrays *cgnn_hybird_partition(int64_t total, const int64_t *vlist, const int64_t *elist,
                                   const float *value, int64_t V) {
    if (total < 0 || V < 0 || V > total || !vlist) {
        set_error("hybird_partition: bad arguments");
        return nullptr;
    }
    return guarded([&] { return hybird_partition(total, vlist, elist, value, V); });
}

cgnn_arrays *cgnn_topo_partition(int64_t R, const int64_t *vlist, const int64_t *elist, const float *value) {
    if (R < 0 || !vlist) {
        set_error("topo_partition: bad arguments");
        return nullptr;
    }
    return guarded([&] { return topo_partition(R, vlist, elist, value); });
}

cgnn_arrays *cgnn_gen_degree(int64_t V, int64_t R, const int64_t *v2v_vlist, const int64_t *v2r_vlist,
                             const int64_t *v2r_elist, const int64_t *r2v_vlist, int levels,
                             const int64_t *const *level_vlists, const int64_t *const *level_elists) {
    // Reference: src/offline/csrc/gen_degree.h:52-82 -- levels are visited from the last
    // to the first, each adding the current degrees of a rule's row entries.
    if (V < 0 || R < 0 || levels < 0) {
        set_error("gen_degree: bad arguments");
        return nullptr;
    }
    return guarded([&] {
        std::vector<i64> vd(V), rd(R);
        for (i64 v = 0; v < V; ++v) vd[v] = v2v_vlist[v + 1] - v2v_vlist[v];
        for (i64 r = 0; r < R; ++r) rd[r] = r2v_vlist[r + 1] - r2v_vlist[r];
        for (int k = levels - 1; k >= 0; --k)
            for (i64 r = 0; r < R; ++r)
                for (i64 e = level_vlists[k][r]; e < level_vlists[k][r + 1]; ++e) rd[r] += rd[level_elists[k][e]];
        for (i64 v = 0; v < V; ++v)
            for (i64 e = v2r_vlist[v]; e < v2r_vlist[v + 1]; ++e) vd[v] += rd[v2r_elist[e]];
        auto *out = new cgnn_arrays;
        out->add(std::move(vd));
        out->add(std::move(rd));
        return out;
    });
}

cgnn_arrays *cgnn_filter_csr(int64_t V, int64_t R, const int64_t *vlist, const int64_t *elist, int threshold) {
    if (V < 0 || R < 0 || !vlist) {
        set_error("filter_csr: bad arguments");
        return nullptr;
    }
    return guarded([&] { return filter_csr(V, R, vlist, elist, threshold); });
}

cgnn_arrays *cgnn_depth_filter_csr(int64_t V, int64_t R, const int64_t *vlist, const int64_t *elist,
                                   int max_depth, int min_edge) {
    if (V < 0 || R < 0 || !vlist) {
        set_error("depth_filter_csr: bad arguments");
        return nullptr;
    }
    return guarded([&] { return depth_filter_csr(V, R, vlist, elist, max_depth, min_edge); });
}

cgnn_arrays *cgnn_gen_vertex_order_csr(int64_t V, int64_t R, const int64_t *vlist, const int64_t *elist) {
    if (V < 0 || R < 0 || !vlist) {
        set_error("gen_vertex_order_csr: bad arguments");
        return nullptr;
    }
    return guarded([&] {
        std::vector<int32_t> order;
        int depth = vertex_order_csr(V, R, vlist, elist, order);
        auto *out = new cgnn_arrays;
        out->add(std::move(order));
        out->scalars.push_back(depth);
        return out;
    });
}

cgnn_arrays *cgnn_gen_vertex_order_csc(int64_t V, int64_t R, const int64_t *vlist, const int64_t *elist) {
    if (V < 0 || R < 0 || !vlist) {
        set_error("gen_vertex_order_csc: bad arguments");
        return nullptr;
    }
    return guarded([&] {
        std::vector<int32_t> order;
        int depth = vertex_order_csc(V, R, vlist, elist, order);
        auto *out = new cgnn_arrays;
        out->add(std::move(order));
        out->scalars.push_back(depth);
        return out;
    });
}

cgnn_arrays *cgnn_add_self_loop_coo(int64_t E, const int64_t *src, const int64_t *dst, int64_t V) {
    // Reference: src/offline/csrc/add_self_loop.h:55-107.  Edges are grouped by ascending
    // source; (v, v) is placed behind v's targets below v unless it is already there.
    // Edges whose source does not come up in that order are left out, as there.
    if (E < 0 || V < 0 || (E > 0 && (!src || !dst))) {
        set_error("add_self_loop_coo: bad arguments");
        return nullptr;
    }
    return guarded([&] {
        std::vector<i64> ns, nd;
        ns.reserve((size_t)(E + V));
        nd.reserve((size_t)(E + V));
        i64 e = 0;
        auto keep = [&] {
            ns.push_back(src[e]);
            nd.push_back(dst[e]);
            ++e;
        };
        for (i64 v = 0; v < V; ++v) {
            while (e < E && src[e] == v && dst[e] < v) keep();
            if (e < E && src[e] == v && dst[e] == v) {
                keep();
            } else {
                ns.push_back(v);
                nd.push_back(v);
            }
            while (e < E && src[e] == v) keep();
        }
        auto *out = new cgnn_arrays;
        out->add(std::move(ns));
        out->add(std::move(nd));
        return out;
    });
}

int cgnn_gcn_norm_coo_compress(int64_t E, const int64_t *src, const int64_t *dst, const float *d, int64_t V,
                               int64_t R, float *weight) {
    // Reference: src/offline/csrc/norm.h:129-166.
    if (E < 0 || V < 0 || R < 0 || (E > 0 && (!src || !dst || !weight)) || (V > 0 && !d)) {
        set_error("gcn_norm_coo_compress: bad arguments");
        return 1;
    }
    for (i64 e = 0; e < E; ++e) {
        const i64 s = src[e], t = dst[e];
        if (s < 0 || t < 0 || s >= V + R || t >= V + R) {
            set_error("gcn_norm_coo_compress: edge %lld out of range", (long long)e);
            return 1;
        }
        if (s < V) weight[e] = t < V ? d[s] * d[t] : d[s];
        else weight[e] = t < V ? d[t] : 1.0f;
    }
    return 0;
}

cgnn_arrays *cgnn_gen_edge_order(int64_t E, const int64_t *src, const int64_t *dst, int64_t V, int64_t R) {
    // Reference: src/offline/csrc/gen_mask.h:10-84.  Phase 0 holds every edge that leaves a
    // vertex.  An edge that leaves a rule is due in the first phase after all rule->rule
    // edges into that rule have been delivered; a rule that only vertices feed is complete
    // after phase 0.  A phase is formed from the state at its start.
    if (E < 0 || V < 0 || R < 0 || (E > 0 && (!src || !dst))) {
        set_error("gen_edge_order: bad arguments");
        return nullptr;
    }
    return guarded([&] {
        std::vector<int32_t> order((size_t)E, -1);
        std::vector<i64> waiting((size_t)R, 0);  // undelivered rule->rule edges into each rule
        std::vector<i64> open;                   // edges that leave a rule, in input order
        for (i64 e = 0; e < E; ++e) {
            if (src[e] < 0 || dst[e] < 0 || src[e] >= V + R || dst[e] >= V + R)
                throw std::runtime_error("gen_edge_order: edge out of range");
            if (src[e] < V) {
                order[e] = 0;
            } else {
                open.push_back(e);
                if (dst[e] >= V) ++waiting[dst[e] - V];
            }
        }
        int phases = 1;
        std::vector<i64> later, delivered;
        while (!open.empty()) {
            later.clear();
            delivered.clear();
            for (i64 e : open) {
                if (waiting[src[e] - V] == 0) {
                    order[e] = phases;
                    if (dst[e] >= V) delivered.push_back(dst[e] - V);
                } else {
                    later.push_back(e);
                }
            }
            if (later.size() == open.size())
                throw std::runtime_error("gen_edge_order: the rule graph has a cycle");
            for (i64 r : delivered) --waiting[r];
            open.swap(later);
            ++phases;
        }
        auto *out = new cgnn_arrays;
        out->add(std::move(order));
        out->scalars.push_back(phases);
        return out;
    });
}

cgnn_arrays *cgnn_compress_csr_batch(int64_t V, const int64_t *vlist, const int64_t *elist, int threads,
                                     int rounds, int min_pair_frequency) {
    (void)threads;
    if (V < 0 || !vlist || rounds < 1) {
        set_error("compress_csr_batch: bad arguments");
        return nullptr;
    }
    if (min_pair_frequency < 3) {
        set_error("compress_csr_batch: min_pair_frequency must be at least 3");
        return nullptr;
    }
    const i64 E = vlist[V];
    if (V >= (i64)INT32_MAX || E >= (i64)INT32_MAX) {
        set_error("compress_csr_batch: CSR array exceeds int32 capacity");
        return nullptr;
    }
    for (i64 e = 0; e < E; ++e)
        if (elist[e] < 0 || elist[e] >= V) {
            set_error("compress_csr_batch: column %lld out of range", (long long)elist[e]);
            return nullptr;
        }
    return guarded([&] { return compress_batch(V, vlist, elist, rounds, min_pair_frequency); });
}

// Columns listed by more rows than this are left out when rows are matched by the columns
// they share: nearly every pair of rows shares such a column (and it stays in cache anyway).
// The limit is halved until matching costs at most kLocalityWork steps per non-zero
// (a column listed by d rows costs d * d steps).
static const i64 kLocalityHubRows = 256;
static const i64 kLocalityWork = 64;

cgnn_arrays *cgnn_csr_locality_order(int64_t rows, const int64_t *vlist, const int64_t *elist) {
    // Rows that gather the same columns should be processed one after the other, so that
    // they find each other's gathers in cache.  Every row is tied to the row it shares most
    // columns with (ties: the lower row); the ties that close no cycle form a forest, and
    // the order is a depth-first walk of it, closest relatives first.  Trees are entered
    // in the lexicographic order of the column lists (shorter list first on a common
    // prefix, then by row number), which also orders the rows that share nothing.
    if (rows < 0 || !vlist || rows >= (i64)INT32_MAX) {
        set_error("csr_locality_order: bad arguments");
        return nullptr;
    }
    return guarded([&] {
        const i64 nnz = vlist[rows];
        std::vector<int32_t> lex((size_t)rows);
        std::iota(lex.begin(), lex.end(), 0);
        auto before = [&](int32_t a, int32_t b) {
            const i64 *pa = elist + vlist[a], *ea = elist + vlist[a + 1];
            const i64 *pb = elist + vlist[b], *eb = elist + vlist[b + 1];
            for (; pa != ea && pb != eb; ++pa, ++pb)
                if (*pa != *pb) return *pa < *pb;
            if ((pa == ea) != (pb == eb)) return pa == ea;
            return a < b;
        };
#ifdef _GLIBCXX_PARALLEL_PARALLEL_H
        __gnu_parallel::sort(lex.begin(), lex.end(), before);
#else
        std::sort(lex.begin(), lex.end(), before);
#endif
        // column -> rows that list it.  Scattered counting and filling are most of the time of
        // this function on graphs beyond the caches, so all cores take part; the rows of a
        // column then stand in no particular order, which the matching below does not read.
        i64 cols = 0, lowest = 0;
#pragma omp parallel for reduction(max : cols) reduction(min : lowest) schedule(static)
        for (i64 e = 0; e < nnz; ++e) {
            cols = std::max(cols, elist[e] + 1);
            lowest = std::min(lowest, elist[e]);
        }
        if (lowest < 0) throw std::runtime_error("csr_locality_order: negative column");
        std::vector<i64> cstart((size_t)cols + 1, 0);
#pragma omp parallel for schedule(static)
        for (i64 e = 0; e < nnz; ++e) __atomic_fetch_add(&cstart[elist[e] + 1], (i64)1, __ATOMIC_RELAXED);
        for (i64 c = 0; c < cols; ++c) cstart[c + 1] += cstart[c];
        std::vector<int32_t> crow((size_t)nnz);
        {
            std::vector<i64> fill(cstart.begin(), cstart.end() - 1);
#pragma omp parallel for schedule(static)
            for (i64 r = 0; r < rows; ++r)
                for (i64 e = vlist[r]; e < vlist[r + 1]; ++e)
                    crow[__atomic_fetch_add(&fill[elist[e]], (i64)1, __ATOMIC_RELAXED)] = (int32_t)r;
        }
        i64 hub_rows = kLocalityHubRows;
        for (; hub_rows > 2; hub_rows /= 2) {
            double steps = 0;
            for (i64 c = 0; c < cols; ++c) {
                const double d = (double)(cstart[c + 1] - cstart[c]);
                if (d <= (double)hub_rows) steps += d * d;
            }
            if (steps <= (double)kLocalityWork * (double)std::max<i64>(nnz, 1)) break;
        }
        // the closest relative of every row
        std::vector<int32_t> best((size_t)rows, -1), shared((size_t)rows, 0);
        // Counting how often every other row turns up: a row with few candidates counts them
        // in a small hash table that stays in the core's cache; only rows with many use the
        // counter per row of the matrix (random accesses into an array of the size of the graph
        // were most of the time of this step).  Both give the same (most, lowest row) answer.
        constexpr int32_t kSlots = 8192, kSmall = kSlots / 2;
#pragma omp parallel
        {
            std::vector<int32_t> count((size_t)rows, 0), touched;
            std::vector<int32_t> key((size_t)kSlots, -1), hits((size_t)kSlots, 0), used;
#pragma omp for schedule(dynamic, 1024)
            for (i64 r = 0; r < rows; ++r) {
                i64 candidates = 0;
                for (i64 e = vlist[r]; e < vlist[r + 1]; ++e) {
                    const i64 d = cstart[elist[e] + 1] - cstart[elist[e]];
                    if (d <= hub_rows) candidates += d;
                }
                int32_t b = -1, most = 0;
                if (candidates <= kSmall) {
                    used.clear();
                    for (i64 e = vlist[r]; e < vlist[r + 1]; ++e) {
                        const i64 c = elist[e];
                        if (cstart[c + 1] - cstart[c] > hub_rows) continue;
                        for (i64 q = cstart[c]; q < cstart[c + 1]; ++q) {
                            const int32_t o = crow[q];
                            if (o == r) continue;
                            uint32_t h = ((uint32_t)o * 2654435761u) >> 19;  // 13 bits: kSlots
                            while (key[h] != o && key[h] != -1) h = (h + 1) & (kSlots - 1);
                            if (key[h] == -1) {
                                key[h] = o;
                                used.push_back((int32_t)h);
                            }
                            ++hits[h];
                        }
                    }
                    for (int32_t h : used) {
                        if (hits[h] > most || (hits[h] == most && key[h] < b)) most = hits[h], b = key[h];
                        key[h] = -1;
                        hits[h] = 0;
                    }
                } else {
                    touched.clear();
                    for (i64 e = vlist[r]; e < vlist[r + 1]; ++e) {
                        const i64 c = elist[e];
                        if (cstart[c + 1] - cstart[c] > hub_rows) continue;
                        for (i64 q = cstart[c]; q < cstart[c + 1]; ++q) {
                            const int32_t o = crow[q];
                            if (o != r && count[o]++ == 0) touched.push_back(o);
                        }
                    }
                    for (int32_t o : touched) {
                        if (count[o] > most || (count[o] == most && o < b)) most = count[o], b = o;
                        count[o] = 0;
                    }
                }
                best[r] = b;
                shared[r] = most;
            }
        }
        // ties that close no cycle, in row order
        std::vector<int32_t> root((size_t)rows);
        std::iota(root.begin(), root.end(), 0);
        auto find = [&](int32_t x) {
            while (root[x] != x) {
                root[x] = root[root[x]];
                x = root[x];
            }
            return x;
        };
        std::vector<char> kept((size_t)rows, 0);
        std::vector<i64> astart((size_t)rows + 1, 0);
        for (i64 r = 0; r < rows; ++r) {
            if (best[r] < 0) continue;
            const int32_t a = find((int32_t)r), c = find(best[r]);
            if (a == c) continue;
            root[a] = c;
            kept[r] = 1;
            ++astart[r + 1];
            ++astart[best[r] + 1];
        }
        for (i64 r = 0; r < rows; ++r) astart[r + 1] += astart[r];
        struct Tie {
            int32_t shared, row;
        };
        std::vector<Tie> adj((size_t)astart[rows]);
        {
            std::vector<i64> fill(astart.begin(), astart.end() - 1);
            for (i64 r = 0; r < rows; ++r)
                if (kept[r]) {
                    adj[fill[r]++] = Tie{shared[r], best[r]};
                    adj[fill[best[r]]++] = Tie{shared[r], (int32_t)r};
                }
        }
#pragma omp parallel for schedule(dynamic, 4096)
        for (i64 r = 0; r < rows; ++r)
            std::sort(adj.begin() + astart[r], adj.begin() + astart[r + 1], [](const Tie &x, const Tie &y) {
                return x.shared != y.shared ? x.shared > y.shared : x.row < y.row;
            });
        // depth-first walk
        std::vector<int32_t> order;
        order.reserve((size_t)rows);
        std::vector<char> seen((size_t)rows, 0);
        std::vector<i64> next(astart.begin(), astart.end() - 1);
        std::vector<int32_t> stack;
        for (i64 i = 0; i < rows; ++i) {
            if (seen[lex[i]]) continue;
            seen[lex[i]] = 1;
            order.push_back(lex[i]);
            stack.push_back(lex[i]);
            while (!stack.empty()) {
                const int32_t top = stack.back();
                if (next[top] == astart[top + 1]) {
                    stack.pop_back();
                    continue;
                }
                const int32_t o = adj[next[top]++].row;
                if (seen[o]) continue;
                seen[o] = 1;
                order.push_back(o);
                stack.push_back(o);
            }
        }
        auto *out = new cgnn_arrays;
        out->add(std::move(order));
        return out;
    });
}

cgnn_arrays *cgnn_csr_fold_levels(int64_t R, const int64_t *vlist, const int64_t *elist, const float *value,
                                  int levels, const int64_t *const *level_vlists,
                                  const int64_t *const *level_elists, const float *const *level_values) {
    // B (R rows) followed by the in-place updates B[r] += sum_c L_k[r, c] * B[c] for k = 0,
    // 1, ... (the rule levels of the compressed propagation, layer/CompressgnnSPMM.py:56-58 of
    // the reference), as one matrix: row r of the result is the row after all updates, its
    // entries merged by column in ascending order.  A level only reads rows that it does not
    // write, so the rows can be rewritten one after the other.
    if (R < 0 || !vlist || levels < 0 || (levels > 0 && (!level_vlists || !level_elists))) {
        set_error("csr_fold_levels: bad arguments");
        return nullptr;
    }
    return guarded([&] {
        typedef std::pair<i64, float> Entry;
        std::vector<std::vector<Entry>> rows((size_t)R);
        for (i64 r = 0; r < R; ++r)
            for (i64 e = vlist[r]; e < vlist[r + 1]; ++e) rows[r].emplace_back(elist[e], value ? value[e] : 1.0f);
        std::vector<Entry> acc;
        for (int k = 0; k < levels; ++k) {
            const i64 *lv = level_vlists[k], *le = level_elists[k];
            const float *lw = level_values ? level_values[k] : nullptr;
            for (i64 r = 0; r < R; ++r) {
                if (lv[r] == lv[r + 1]) continue;
                acc = rows[r];
                for (i64 e = lv[r]; e < lv[r + 1]; ++e) {
                    const i64 c = le[e];
                    if (c < 0 || c >= R) throw std::runtime_error("csr_fold_levels: level column out of range");
                    if (lv[c] != lv[c + 1]) throw std::runtime_error("csr_fold_levels: a level reads a row that it writes");
                    const float w = lw ? lw[e] : 1.0f;
                    for (const Entry &x : rows[c]) acc.emplace_back(x.first, w * x.second);
                }
                std::stable_sort(acc.begin(), acc.end(), [](const Entry &a, const Entry &b) { return a.first < b.first; });
                std::vector<Entry> merged;
                for (const Entry &x : acc) {
                    if (!merged.empty() && merged.back().first == x.first) merged.back().second += x.second;
                    else merged.push_back(x);
                }
                rows[r].swap(merged);
            }
        }
        std::vector<i64> nv((size_t)R + 1, 0), ne;
        std::vector<float> nw;
        for (i64 r = 0; r < R; ++r) {
            nv[r + 1] = nv[r] + (i64)rows[r].size();
            for (const Entry &x : rows[r]) {
                ne.push_back(x.first);
                nw.push_back(x.second);
            }
        }
        auto *out = new cgnn_arrays;
        out->add(std::move(nv));
        out->add(std::move(ne));
        out->add(std::move(nw));
        return out;
    });
}

cgnn_arrays *cgnn_csr_permute_rows(int64_t rows, const int64_t *vlist, const int64_t *elist, const float *value,
                                   const int32_t *order) {
    if (rows < 0 || !vlist || (rows > 0 && !order)) {
        set_error("csr_permute_rows: bad arguments");
        return nullptr;
    }
    return guarded([&] {
        std::vector<i64> nv((size_t)rows + 1, 0), ne((size_t)vlist[rows]);
        std::vector<float> nw(value ? (size_t)vlist[rows] : 0);
        for (i64 g = 0; g < rows; ++g) {
            const i64 r = order[g];
            if (r < 0 || r >= rows) throw std::runtime_error("csr_permute_rows: order is not a permutation");
            nv[g + 1] = nv[g] + (vlist[r + 1] - vlist[r]);
        }
        if (nv[rows] != vlist[rows]) throw std::runtime_error("csr_permute_rows: order is not a permutation");
#pragma omp parallel for schedule(static)
        for (i64 g = 0; g < rows; ++g) {
            const i64 r = order[g];
            std::copy(elist + vlist[r], elist + vlist[r + 1], ne.begin() + nv[g]);
            if (value) std::copy(value + vlist[r], value + vlist[r + 1], nw.begin() + nv[g]);
        }
        auto *out = new cgnn_arrays;
        out->add(std::move(nv));
        out->add(std::move(ne));
        out->add(std::move(nw));
        return out;
    });
}

cgnn_arrays *cgnn_csr_hstack(int64_t rows, const int64_t *vlist0, const int64_t *elist0, const float *value0,
                             const int64_t *vlist1, const int64_t *elist1, const float *value1, int64_t col_offset) {
    if (rows < 0 || !vlist0 || !vlist1) {
        set_error("csr_hstack: bad arguments");
        return nullptr;
    }
    return guarded([&] {
        const i64 n0 = vlist0[rows], n1 = vlist1[rows];
        std::vector<i64> ptr(rows + 1, 0), col;
        std::vector<float> val;
        col.reserve(n0 + n1);
        val.reserve(n0 + n1);
        for (i64 r = 0; r < rows; ++r) {
            for (i64 e = vlist0[r]; e < vlist0[r + 1]; ++e) {
                col.push_back(elist0[e]);
                val.push_back(value0[e]);
            }
            for (i64 e = vlist1[r]; e < vlist1[r + 1]; ++e) {
                col.push_back(elist1[e] + col_offset);
                val.push_back(value1[e]);
            }
            ptr[r + 1] = (i64)col.size();
        }
        auto *out = new cgnn_arrays;
        out->add(std::move(ptr));
        out->add(std::move(col));
        out->add(std::move(val));
        return out;
    });
}

int cgnn_csr_row_stats(int64_t rows, const int64_t *vlist, int64_t *max_row, int64_t hist[40]) {
    if (rows < 0 || !vlist) {
        set_error("csr_row_stats: bad arguments");
        return 1;
    }
    i64 mx = 0;
    for (int k = 0; k < 40; ++k) hist[k] = 0;
    for (i64 r = 0; r < rows; ++r) {
        const i64 len = vlist[r + 1] - vlist[r];
        mx = std::max(mx, len);
        int k = 0;
        while (((i64)1 << k) <= len) ++k;  // len in [2^(k-1), 2^k)
        ++hist[k];
    }
    if (max_row) *max_row = mx;
    return 0;
}

cgnn_arrays *cgnn_gen_chung_lu(int64_t V, int64_t target_edges, double exponent, uint64_t seed) {
    if (V < 0 || target_edges < 0 || exponent <= 1.0) {
        set_error("gen_chung_lu: bad arguments");
        return nullptr;
    }
    return guarded([&] { return gen_chung_lu(V, target_edges, exponent, seed); });
}

cgnn_arrays *cgnn_gen_copy_model(int64_t V, double avg_degree, double copy_prob, uint64_t seed) {
    if (V < 0 || avg_degree < 0 || copy_prob < 0 || copy_prob > 1) {
        set_error("gen_copy_model: bad arguments");
        return nullptr;
    }
    return guarded([&] { return gen_copy_model(V, avg_degree, copy_prob, seed); });
}

}  // extern "C"
