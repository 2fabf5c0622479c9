// CSR SpMM for gfx950 (wave64): Y (+)= A * X with dense row-major X, Y of width F.
//
// Geometry shared by all kernels here.  A "lane group" of LPR consecutive lanes
// (LPR a power of two, 4..64) owns one output row at a time; lane l of the group
// holds VEC consecutive features starting at (tile*LPR + l)*VEC for TILES tiles, so a
// group reads and writes LPR*VEC*sizeof(T) contiguous bytes per tile (512 B per wave
// instruction when VEC*sizeof(T) = 16, i.e. global_load_dwordx4 on every lane).
// Features beyond LPR*VEC*TILES are covered by blockIdx.y.
//
// The entries of a row (column, value, row) are loaded once per lane group, one entry per
// lane with a coalesced load, and handed to all lanes of the group through the LDS
// crossbar (ds_bpermute); the gathers of a round are issued together, none behind the end
// of the row.  Loading every entry in every lane made the kernels bound by vector
// instruction issue (address arithmetic), not by memory.
//
// Two schedules:
//   * row schedule  -- a lane group per row, entries summed in ascending order; the
//     result is bit-identical to the sequential CPU sum of the reference
//     (src/runtime/csrc/sparse/cpu/spmm_cpu.cpp:48-68): products and sums are rounded
//     separately (this file is built with -ffp-contract=off).
//   * nnz schedule  -- a lane group per run of about seg_nnz consecutive non-zeros (rows
//     of any length cost the same).  Rows of at most seg_nnz entries always lie inside
//     one run and are summed exactly as in the row schedule.  Longer rows are cut at
//     multiples of seg_nnz: the part that continues into the next run is a carry.  The
//     lane groups of one workgroup first add their carries of the same row in LDS, in
//     ascending order, so at most one carry row per output row and workgroup reaches
//     memory.  spmm_carry_reduce_kernel sums the carries of very long rows 64 at a
//     time, level by level (a row with a million entries is not walked by one lane
//     group), and spmm_fixup_kernel adds what is left, in ascending order.
//     Every output element receives its additions in a fixed order (where an atomic add
//     is used it is the only addition to that element), so results are reproducible run
//     to run.
//
// Modes: VAL (stored values), UNIT (all values 1), RELU_MASK (unit values, gathered
// rows zeroed where a second matrix is <= 0), DUAL (columns below `split` gather from
// X, the others from X1; the two partial sums are kept apart and combined as
// (0 + sum1) + sum0, which is what two successive accumulating products give).
//
// X may alias Y when accumulating (rule levels are updated in place, reference
// layer/CompressgnnSPMM.py:56-58), so X and Y carry no __restrict__; a row that is
// written is never gathered in the same launch (levels only read earlier levels).
#include <mutex>
#include <type_traits>

#include "common.h"

namespace cgnn {
namespace {

constexpr int kUnroll = 4;        // gathers in flight per lane and tile, nnz schedule (with 7 waves per SIMD;
                                  // 8 in flight with 5 waves measured the same)
constexpr int kRowUnroll = 4;     // same for the row schedule (8: 9 % slower on web-graph out-lists, 2: 13 %, 16: 38 %)
constexpr int kXcds = 8;          // accelerator dies of an MI355X, each with its own L2
constexpr int kDefaultSeg = 64;   // non-zeros per lane group in the nnz schedule

enum { MODE_VAL = 0, MODE_UNIT = 1, MODE_RELU_MASK = 2, MODE_DUAL = 3, MODE_SIGN_MASK = 4 };

template <typename T, int VEC>
struct alignas(sizeof(T) * VEC) Pack {
    T v[VEC];
};

template <typename T>
struct SpmmArgs {
    const int32_t *rowptr;
    const int32_t *colidx;
    const int32_t *rowidx;
    const int32_t *rowmap;  // row schedule: stored row g is row rowmap[g] of Y (or NULL)
    const T *val;
    const T *X;   // gathered matrix (may alias Y)
    const T *X1;  // MODE_DUAL: source of the columns >= split
    const T *M;   // MODE_RELU_MASK: rows of X are zeroed where M <= 0
    const uint32_t *signs;  // MODE_SIGN_MASK: the same with one bit per element (set: keep), sign_words words per row
    int32_t sign_words;
    T *Y;
    int32_t *carry_row;  // [nseg] row a run carries into, or -1
    T *carry;            // [nseg x F]
    int32_t *carry_row_out;  // spmm_carry_reduce_kernel: the next, 32 times shorter level
    T *carry_out;
    int64_t F;
    int32_t rows;
    int32_t nnz;
    int32_t nseg;
    int32_t seg_nnz;
    int32_t split;
    int32_t accumulate;
    // Runs per workgroup of the nnz kernel that wrote carry_row/carry (its carries are
    // merged per workgroup: see kMerged), or 1 for the plain list a reduction level writes.
    int32_t merge_stride;
    int32_t stretch_log2;  // log2 of the workgroups per XCD stretch (see logical_block); set at launch
    int32_t blocks;        // workgroups with work (the grid rounds this up to a multiple of kXcds)
    int32_t read_once;     // MODE_UNIT: every row of X is gathered once (member lists), so with streaming loads
    const int32_t *cut_rows;    // spmm_fixup_rows_kernel: the stored rows that the runs cut, ascending
    const int32_t *empty_rows;  // and the stored rows without entries
    int32_t n_cut_rows, n_empty_rows;
    const int32_t *run_start;   // nnz schedule: first non-zero of every run, [nseg + 1], or NULL (run_boundary)
};

// carry_row values below zero: the run carries nothing, or its carry was added to that
// of an earlier run of the same workgroup (the row of Y is the one of that earlier run).
constexpr int kNoCarry = -1;
constexpr int kMerged = -2;

template <typename T, int VEC>
__device__ __forceinline__ Pack<T, VEC> load_pack(const T *p) {
    return *reinterpret_cast<const Pack<T, VEC> *>(p);
}
// Streaming load for rows that this launch reads once.
template <typename T, int VEC>
__device__ __forceinline__ Pack<T, VEC> load_pack_stream(const T *p) {
    Pack<T, VEC> x;
    if constexpr (VEC == 1) {
        x.v[0] = __builtin_nontemporal_load(p);
    } else {
        typedef T vec_t __attribute__((ext_vector_type(VEC)));
        const vec_t v = __builtin_nontemporal_load(reinterpret_cast<const vec_t *>(p));
#pragma unroll
        for (int i = 0; i < VEC; ++i) x.v[i] = v[i];
    }
    return x;
}
template <typename T, int VEC>
__device__ __forceinline__ void store_pack(T *p, const Pack<T, VEC> &x) {
    *reinterpret_cast<Pack<T, VEC> *>(p) = x;
}
// Streaming store for rows that are written once and not read again by this launch.
template <typename T, int VEC>
__device__ __forceinline__ void store_pack_stream(T *p, const Pack<T, VEC> &x) {
    if constexpr (VEC == 1) {
        __builtin_nontemporal_store(x.v[0], p);
    } else {
        typedef T vec_t __attribute__((ext_vector_type(VEC)));
        vec_t v;
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[i] = x.v[i];
        __builtin_nontemporal_store(v, reinterpret_cast<vec_t *>(p));
    }
}

// Per-lane feature offsets of the TILES tiles; foff[t] < 0 marks a tile beyond F.
template <int VEC, int LPR, int TILES>
__device__ __forceinline__ void feature_offsets(int64_t F, int lane, int64_t foff[TILES]) {
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
        int64_t f = ((int64_t)(blockIdx.y * TILES + t) * LPR + lane) * VEC;
        foff[t] = f < F ? f : -1;
    }
}

// Accumulator of one output row.  MODE_DUAL keeps the sums over the two sources apart: the
// entries of a row are sorted by column, so those of the first source come first; when the
// first entry of the second source arrives the running sum is put aside and started anew.
template <typename T, int VEC, int TILES, int MODE>
struct Acc {
    Pack<T, VEC> a0[TILES];                          // running sum
    Pack<T, VEC> a1[MODE == MODE_DUAL ? TILES : 1];  // MODE_DUAL: finished sum over the first source
    bool second_source;                              // MODE_DUAL: a1 is in use

    __device__ __forceinline__ void clear() {
        second_source = false;
#pragma unroll
        for (int t = 0; t < TILES; ++t)
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                a0[t].v[i] = T(0);
                if constexpr (MODE == MODE_DUAL) a1[t].v[i] = T(0);
            }
    }
    // entry with gathered tiles x, value w, from source `src` (0 or 1)
    __device__ __forceinline__ void add(const Pack<T, VEC> x[TILES], T w, int src) {
        if constexpr (MODE == MODE_DUAL) {
            // At most once per row, so the whole wave jumps over it nearly always.  Written
            // with value selects under a wave-uniform branch: a branch per lane would be
            // turned into selects on every entry.
            const bool change = src != 0 && !second_source;
            if (__ballot(change)) {
#pragma unroll
                for (int t = 0; t < TILES; ++t)
#pragma unroll
                    for (int i = 0; i < VEC; ++i) {
                        a1[t].v[i] = change ? a0[t].v[i] : a1[t].v[i];
                        a0[t].v[i] = change ? T(0) : a0[t].v[i];
                    }
                second_source = second_source || change;
            }
        }
#pragma unroll
        for (int t = 0; t < TILES; ++t)
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                if constexpr (MODE == MODE_VAL || MODE == MODE_DUAL) a0[t].v[i] = a0[t].v[i] + x[t].v[i] * w;
                else a0[t].v[i] = a0[t].v[i] + x[t].v[i];
            }
    }
    // the row's value on top of `base`: (base + sum1) + sum0 in MODE_DUAL, base + sum otherwise
    __device__ __forceinline__ T total(T base, int t, int i) const {
        if constexpr (MODE == MODE_DUAL) {
            const T sum0 = second_source ? a1[t].v[i] : a0[t].v[i];
            const T sum1 = second_source ? a0[t].v[i] : T(0);
            return (base + sum1) + sum0;
        } else {
            return base + a0[t].v[i];
        }
    }
};

// Y[row] = (accumulate ? Y[row] : 0) + acc
template <typename T, int VEC, int TILES, int MODE>
__device__ __forceinline__ void write_row(T *Y, int64_t F, int row, const int64_t foff[TILES],
                                          const Acc<T, VEC, TILES, MODE> &acc, int accumulate) {
    T *yrow = Y + (int64_t)row * F;
    // Only the plain product (MODE_VAL) can add to an existing Y.  The other modes write every row once, and
    // knowing that at compile time keeps a load of Y out of the block that closes a row inside a run of the
    // nnz schedule, where the compiler would have to wait for it on every path behind the block.
    if constexpr (MODE != MODE_VAL) accumulate = 0;
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
        if (foff[t] < 0) continue;
        Pack<T, VEC> o;
        if (accumulate) {
            o = load_pack<T, VEC>(yrow + foff[t]);
        } else {
#pragma unroll
            for (int i = 0; i < VEC; ++i) o.v[i] = T(0);
        }
#pragma unroll
        for (int i = 0; i < VEC; ++i) o.v[i] = acc.total(o.v[i], t, i);
        if (accumulate) store_pack<T, VEC>(yrow + foff[t], o);
        else store_pack_stream<T, VEC>(yrow + foff[t], o);
    }
}

// Gather one feature tile of column c (source chosen by `src` in MODE_DUAL, masked by
// M in MODE_RELU_MASK and by the bits of `signs` in MODE_SIGN_MASK).
template <typename T, int VEC, int MODE>
__device__ __forceinline__ Pack<T, VEC> gather(const SpmmArgs<T> &a, int c, int src, int64_t foff) {
    Pack<T, VEC> x;
    if (foff < 0) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) x.v[i] = T(0);
        return x;
    }
    const T *base = a.X;
    if constexpr (MODE == MODE_DUAL) {
        // both pointers are read first and chosen between as values (a choice between the two
        // fields of the argument block becomes a vector load of the chosen field, and a wait)
        const T *first = a.X, *second = a.X1;
        base = src ? second : first;
        c -= src ? a.split : 0;
    }
    const int64_t off = (int64_t)c * (int32_t)a.F + foff;  // F < 2^31: one 32 x 32 -> 64 bit multiply
    // rows that are gathered once (member lists; masks exist for those only) are not kept in the caches
    if (MODE == MODE_RELU_MASK || MODE == MODE_SIGN_MASK || (MODE == MODE_UNIT && a.read_once))
        x = load_pack_stream<T, VEC>(base + off);
    else
        x = load_pack<T, VEC>(base + off);
    if constexpr (MODE == MODE_SIGN_MASK) {
        // VEC divides 32, so the bits of one pack lie in one word
        const uint32_t bits = a.signs[(int64_t)c * a.sign_words + (foff >> 5)] >> (foff & 31);
#pragma unroll
        for (int i = 0; i < VEC; ++i) x.v[i] = ((bits >> i) & 1u) ? x.v[i] : T(0);
    }
    if constexpr (MODE == MODE_RELU_MASK) {
        Pack<T, VEC> m = load_pack_stream<T, VEC>(a.M + off);
#pragma unroll
        for (int i = 0; i < VEC; ++i) x.v[i] = (m.v[i] <= T(0)) ? T(0) : x.v[i];
    }
    return x;
}

// Row of Y that stored row r stands for.
template <typename T>
__device__ __forceinline__ int out_row(const SpmmArgs<T> &a, int r) {
    return a.rowmap != nullptr ? a.rowmap[r] : r;
}

// Workgroups are dealt to the XCDs round robin.  XCD x takes every kXcds-th stretch of
// consecutive workgroups' worth of stored rows (or runs): rows that follow each other in the
// store (a locality order, or a natural order that has locality) meet in one L2, and every
// XCD gets the same mix of the matrix (one contiguous share each would leave the XCD with the
// least reuse to finish last).  A stretch holds kXcdStretchGroups lane groups, about what an
// XCD holds at a time at F = 128, so an XCD works on one region of the order at once (a
// quarter and twice that measured 1.5 % slower on the web graph, four times 20 %: too few
// stretches to even out).  Small launches take shorter stretches, at least
// kMinStretchesPerXcd per XCD.
constexpr int kXcdStretchGroups = 2048;
constexpr int kMinStretchesPerXcd = 6;

template <int GPB>
constexpr int xcd_stretch() {
    return kXcdStretchGroups / GPB > 0 ? kXcdStretchGroups / GPB : 1;
}

// log2 of the stretch (in workgroups) for a launch of `blocks` workgroups of GPB lane groups
template <int GPB>
int stretch_log2_for(int64_t blocks) {
    int lg = 0;
    while ((2 << lg) <= xcd_stretch<GPB>()) ++lg;
    while (lg > 0 && blocks < ((int64_t)kXcds * kMinStretchesPerXcd << lg)) --lg;
    return lg;
}

// Whole rounds of kXcds stretches are dealt first; what is left over is dealt the same way in
// stretches half as long, and so on down to single workgroups, so that no XCD is left with a
// whole stretch more than another.
template <typename T>
__device__ __forceinline__ int logical_block(const SpmmArgs<T> &a) {
    const int xcd = blockIdx.x % kXcds;
    int turn = blockIdx.x / kXcds;  // this workgroup's number on its XCD
    int base = 0, left = a.blocks;
    for (int lg = a.stretch_log2; lg > 0; --lg) {
        const int share = (left >> (lg + 3)) << lg;  // workgroups per XCD dealt in stretches of 2^lg  (kXcds = 2^3)
        if (turn < share) return base + ((((turn >> lg) * kXcds) + xcd) << lg) + (turn & ((1 << lg) - 1));
        turn -= share;
        base += share * kXcds;
        left -= share * kXcds;
    }
    return base + turn * kXcds + xcd;
}

// ---------------------------------------------------------------- row schedule --
template <typename T, int VEC, int LPR, int TILES, int MODE>
__global__ __launch_bounds__(kBlock) void spmm_row_kernel(SpmmArgs<T> a) {
    constexpr int GPB = kBlock / LPR;
    const int lane = threadIdx.x % LPR;
    int row = logical_block(a) * GPB + threadIdx.x / LPR;
    if constexpr (LPR == kWave) row = __builtin_amdgcn_readfirstlane(row);
    if (row >= a.rows) return;
    const int e0 = a.rowptr[row], e1 = a.rowptr[row + 1];
    row = out_row(a, row);  // from here on: the row of Y
    int64_t foff[TILES];
    feature_offsets<VEC, LPR, TILES>(a.F, lane, foff);
    Acc<T, VEC, TILES, MODE> acc;
    acc.clear();
    if (e0 == e1) {
        if (!a.accumulate) write_row<T, VEC, TILES, MODE>(a.Y, a.F, row, foff, acc, 0);
        return;
    }
    if constexpr (sizeof(T) == 4) {
        constexpr int RU = LPR < kRowUnroll ? LPR : kRowUnroll;  // entries per round: no more than lanes to stage them
        // The lanes of the group load one entry each (one coalesced load per array for LPR
        // entries), and every entry is then handed to all lanes through the LDS crossbar:
        // no address arithmetic and no memory instruction per entry and lane for the indices.
        const int group_lane0 = 4 * ((threadIdx.x % kWave) - lane);  // byte address of the group's first lane
        // lanes beyond the width gather feature 0 again (never stored): no test per gather
        int64_t fld[TILES];
#pragma unroll
        for (int t = 0; t < TILES; ++t) fld[t] = foff[t] < 0 ? 0 : foff[t];
        for (int e = e0; e < e1; e += LPR) {
            int my_c = 0;
            T my_w = T(1);
            if (e + lane < e1) {
                my_c = a.colidx[e + lane];
                if (a.val) my_w = a.val[e + lane];
            }
            const int cnt = min(e1 - e, LPR);
            for (int u0 = 0; u0 < cnt; u0 += RU) {
                int c[RU];
                T w[RU];
#pragma unroll
                for (int u = 0; u < RU; ++u) {
                    const int from = group_lane0 + 4 * (u0 + u);
                    c[u] = __builtin_amdgcn_ds_bpermute(from, my_c);
                    w[u] = __builtin_bit_cast(T, __builtin_amdgcn_ds_bpermute(from, __builtin_bit_cast(int, my_w)));
                }
                // Entries of the second source are rare (columns that stand for rules): when the
                // wave has none in this round, the gathers need no choice of source per lane.
                bool second = false;
                if constexpr (MODE == MODE_DUAL) {
#pragma unroll
                    for (int u = 0; u < RU; ++u) second = second || (u0 + u < cnt && c[u] >= a.split);
                }
                auto gather_and_add = [&](auto plain) {
                    constexpr bool kPlain = decltype(plain)::value;  // every entry from the first source
                    Pack<T, VEC> x[RU][TILES];
#pragma unroll
                    for (int u = 0; u < RU; ++u)
                        if (u0 + u < cnt) {  // no gathers behind the row's end: repeated ones still cost issue slots
#pragma unroll
                            for (int t = 0; t < TILES; ++t)
                                x[u][t] = gather<T, VEC, MODE>(a, c[u], kPlain ? 0 : c[u] >= a.split, fld[t]);
                        }
#pragma unroll
                    for (int u = 0; u < RU; ++u)
                        if (u0 + u < cnt) acc.add(x[u], w[u], kPlain ? 0 : c[u] >= a.split);
                };
                if (MODE != MODE_DUAL || __ballot(second) == 0) gather_and_add(std::true_type{});
                else gather_and_add(std::false_type{});
            }
        }
    } else {
        for (int e = e0; e < e1; e += kRowUnroll) {
            int c[kRowUnroll];
            T w[kRowUnroll];
            Pack<T, VEC> x[kRowUnroll][TILES];
#pragma unroll
            for (int u = 0; u < kRowUnroll; ++u) {
                const int idx = min(e + u, e1 - 1);
                c[u] = a.colidx[idx];
                w[u] = a.val ? a.val[idx] : T(1);
            }
#pragma unroll
            for (int u = 0; u < kRowUnroll; ++u)
                if (e + u < e1) {
#pragma unroll
                    for (int t = 0; t < TILES; ++t) x[u][t] = gather<T, VEC, MODE>(a, c[u], c[u] >= a.split, foff[t]);
                }
#pragma unroll
            for (int u = 0; u < kRowUnroll; ++u)
                if (e + u < e1) acc.add(x[u], w[u], c[u] >= a.split);
        }
    }
    write_row<T, VEC, TILES, MODE>(a.Y, a.F, row, foff, acc, a.accumulate);
}

// ---------------------------------------------------------------- nnz schedule --
// Run s covers the non-zeros [run_boundary(s*K), run_boundary((s+1)*K)).  A boundary
// that falls inside a row of at most K entries is moved back to the start of that row,
// so such rows are never split (and are summed in the same order as the row schedule);
// only rows longer than K are cut, at multiples of K.  Runs hold fewer than 2K entries.
template <typename T>
__device__ __forceinline__ int run_boundary(const SpmmArgs<T> &a, int e) {
    if (e >= a.nnz) return a.nnz;
    const int r = a.rowidx[e];
    const int s0 = a.rowptr[r];
    return (a.rowptr[r + 1] - s0 <= a.seg_nnz) ? s0 : e;
}

template <typename T, int VEC, int LPR, int TILES, int MODE>
__global__ __launch_bounds__(kBlock, (TILES == 1 && LPR >= 16) ? 7 : 1) void spmm_nnz_kernel(SpmmArgs<T> a) {
    constexpr int GPB = kBlock / LPR;
    __shared__ int wg_row[GPB];
    __shared__ Pack<T, VEC> wg_carry[TILES][kBlock];
    const int lane = threadIdx.x % LPR, grp = threadIdx.x / LPR;
    int seg = logical_block(a) * GPB + grp;
    if constexpr (LPR == kWave) seg = __builtin_amdgcn_readfirstlane(seg);
    int e0 = 0, e1 = 0;
    if (seg < a.nseg) {
        if (a.run_start != nullptr) {  // one load instead of two dependent ones
            e0 = a.run_start[seg];
            e1 = a.run_start[seg + 1];
        } else {
            e0 = run_boundary(a, seg * a.seg_nnz);
            e1 = run_boundary(a, (seg + 1) * a.seg_nnz);
        }
    }
    // e0 >= e1 inside the list cannot happen for a well-formed CSR
    const bool active = e0 < e1;
    int64_t foff[TILES];
    feature_offsets<VEC, LPR, TILES>(a.F, lane, foff);
    Acc<T, VEC, TILES, MODE> acc;
    acc.clear();
    int cur = -1;
    bool continues = false;
    if (active) {
        // A run names its rows by the row of Y they are written to (rowmap[stored row], which the
        // lanes look up beside their entries), so that closing a row inside the run needs no load
        // of its own: a load there, and the wait for it, would stand between the gathers of the run.
        // The two-source product over rows of 512 bytes and more keeps the other form -- the run names
        // its rows by their stored number and looks the row of Y up where a row ends.  The look-up
        // beside the entries puts one more load between a run's entries and its first gathers and
        // holds two more values per lane in a kernel that sits at its register limit (72 for seven
        // waves per SIMD): the F = 128 kernel, bound by its traffic either way, took 221 us with it
        // and takes 213 us without (F = 16: 76 -> 62 us with it; the 18.5 M-vertex graph at F = 64:
        // 13.6 -> 13.4 ms; the mask modes, which have no rowmap, lose the wait and nothing else).
        constexpr bool kNamesRowsOfY = !(MODE == MODE_DUAL && VEC * LPR * sizeof(T) >= 512);
        auto named = [&](int stored_row) { return kNamesRowsOfY ? out_row(a, stored_row) : stored_row; };
        auto row_of_y = [&](int name) { return kNamesRowsOfY ? name : out_row(a, name); };
        int cur_out;
        // looked at when the run is done: the stored row of the last entry (the row a carry belongs
        // to) and the row of the entry behind the run; asked for beside the entries
        int last_row, row_behind;
        if constexpr (!kNamesRowsOfY) {  // the names are the stored rows: the first is read here, the last is at hand at the end
            cur_out = a.rowidx[e0];
            row_behind = e1 < a.nnz ? a.rowidx[e1] : -1;
        }
        if constexpr (LPR >= kUnroll && sizeof(T) == 4) {
            // As in the row schedule: the lanes of the group load one entry each, and the
            // entries reach all lanes through the LDS crossbar.
            const int group_lane0 = 4 * ((threadIdx.x % kWave) - lane);
            int64_t fld[TILES];  // lanes beyond the width gather feature 0 again (never stored)
#pragma unroll
            for (int t = 0; t < TILES; ++t) fld[t] = foff[t] < 0 ? 0 : foff[t];
            for (int e = e0; e < e1; e += LPR) {
                int my_o = 0, my_c = 0;
                T my_w = T(1);
                if (e + lane < e1) {
                    my_o = named(a.rowidx[e + lane]);
                    my_c = a.colidx[e + lane];
                    if constexpr (MODE == MODE_DUAL) my_w = a.val[e + lane];
                    if constexpr (MODE == MODE_VAL) my_w = a.val != nullptr ? a.val[e + lane] : T(1);
                }
                if constexpr (kNamesRowsOfY) {
                    // with every batch of entries, so that no load of the run waits for another but
                    // the row numbers for their rows (the same two words each time)
                    last_row = a.rowidx[e1 - 1];
                    row_behind = e1 < a.nnz ? a.rowidx[e1] : -1;
                    // the run begins with the row of its first entry
                    const int batch_first = __builtin_amdgcn_ds_bpermute(group_lane0, my_o);
                    if (e == e0) cur_out = batch_first;
                }
                const int cnt = min(e1 - e, LPR);
                for (int u0 = 0; u0 < cnt; u0 += kUnroll) {
                    int o[kUnroll], c[kUnroll];
                    T w[kUnroll];
#pragma unroll
                    for (int u = 0; u < kUnroll; ++u) {
                        const int from = group_lane0 + 4 * (u0 + u);
                        o[u] = __builtin_amdgcn_ds_bpermute(from, my_o);
                        c[u] = __builtin_amdgcn_ds_bpermute(from, my_c);
                        if constexpr (MODE == MODE_VAL || MODE == MODE_DUAL)
                            w[u] = __builtin_bit_cast(T, __builtin_amdgcn_ds_bpermute(from, __builtin_bit_cast(int, my_w)));
                        else
                            w[u] = T(1);
                    }
                    // Lanes without an entry hold column 0 (a row of X like any other) and value 1, and
                    // positions behind the last entry of a batch read those: a round may gather for them,
                    // nothing is added for them.  Only a block without first-source columns sees such a
                    // position as one of the second source, and takes the slower path for that round.
                    bool second = false;
                    if constexpr (MODE == MODE_DUAL) {
#pragma unroll
                        for (int u = 0; u < kUnroll; ++u) second = second | (c[u] >= a.split);
                    }
                    auto gather_and_add = [&](auto plain) {
                        constexpr bool kPlain = decltype(plain)::value;  // every entry from the first source
                        Pack<T, VEC> x[kUnroll][TILES];
                        // Up to 64 bytes per lane group and gather, a position behind the last entry gathers
                        // like the others (column 0, see above): the branches around four small loads cost
                        // more than the loads.  Wider rows skip it: there the extra row is what costs.
                        constexpr bool kGatherAll = VEC * LPR * sizeof(T) <= 64;
#pragma unroll
                        for (int u = 0; u < kUnroll; ++u)
                            if (kGatherAll || u0 + u < cnt) {
#pragma unroll
                                for (int t = 0; t < TILES; ++t)
                                    x[u][t] = gather<T, VEC, MODE>(a, c[u], kPlain ? 0 : c[u] >= a.split, fld[t]);
                            }
#pragma unroll
                        for (int u = 0; u < kUnroll; ++u) {
                            if (u0 + u < cnt) {
                                if (o[u] != cur_out) {
                                    // the row ends inside this run: finish it here
                                    write_row<T, VEC, TILES, MODE>(a.Y, a.F, row_of_y(cur_out), foff, acc, a.accumulate);
                                    acc.clear();
                                    cur_out = o[u];
                                }
                                acc.add(x[u], w[u], kPlain ? 0 : c[u] >= a.split);
                            }
                        }
                    };
                    if (MODE != MODE_DUAL || __ballot(second) == 0) gather_and_add(std::true_type{});
                    else gather_and_add(std::false_type{});
                }
            }
        } else {
            if constexpr (kNamesRowsOfY) {
                cur_out = named(a.rowidx[e0]);
                last_row = a.rowidx[e1 - 1];
                row_behind = e1 < a.nnz ? a.rowidx[e1] : -1;
            }
            for (int e = e0; e < e1; e += kUnroll) {
                int o[kUnroll], c[kUnroll];
                T w[kUnroll];
                Pack<T, VEC> x[kUnroll][TILES];
#pragma unroll
                for (int u = 0; u < kUnroll; ++u) {
                    const int idx = min(e + u, e1 - 1);
                    o[u] = named(a.rowidx[idx]);
                    c[u] = a.colidx[idx];
                    if constexpr (MODE == MODE_DUAL) w[u] = a.val[idx];
                    else if constexpr (MODE == MODE_VAL) w[u] = a.val != nullptr ? a.val[idx] : T(1);
                    else w[u] = T(1);
                }
#pragma unroll
                for (int u = 0; u < kUnroll; ++u)
                    if (e + u < e1) {
#pragma unroll
                        for (int t = 0; t < TILES; ++t)
                            x[u][t] = gather<T, VEC, MODE>(a, c[u], c[u] >= a.split, foff[t]);
                    }
#pragma unroll
                for (int u = 0; u < kUnroll; ++u) {
                    if (e + u < e1) {
                        if (o[u] != cur_out) {
                            // the row ends inside this run: finish it here
                            write_row<T, VEC, TILES, MODE>(a.Y, a.F, row_of_y(cur_out), foff, acc, a.accumulate);
                            acc.clear();
                            cur_out = o[u];
                        }
                        acc.add(x[u], w[u], c[u] >= a.split);
                    }
                }
            }
        }
        cur = kNamesRowsOfY ? last_row : cur_out;
        continues = row_behind == cur;
        if (!continues) write_row<T, VEC, TILES, MODE>(a.Y, a.F, row_of_y(cur_out), foff, acc, a.accumulate);
    }
    // The carries of one row are added per workgroup: the first of its lane groups that
    // carries the row takes those of the groups behind it, in ascending order.
    Pack<T, VEC> part[TILES];
#pragma unroll
    for (int t = 0; t < TILES; ++t)
#pragma unroll
        for (int i = 0; i < VEC; ++i) part[t].v[i] = acc.total(T(0), t, i);
    if (lane == 0) wg_row[grp] = continues ? cur : kNoCarry;
    if (continues) {
#pragma unroll
        for (int t = 0; t < TILES; ++t) wg_carry[t][threadIdx.x] = part[t];
    }
    __syncthreads();
    if (seg >= a.nseg) return;
    int mark = kNoCarry;
    if (continues) {
        const bool first = grp == 0 || wg_row[grp - 1] != cur;
        mark = first ? cur : kMerged;
        if (first) {
            for (int g = grp + 1; g < GPB && wg_row[g] == cur; ++g)
#pragma unroll
                for (int t = 0; t < TILES; ++t) {
                    const Pack<T, VEC> o = wg_carry[t][g * LPR + lane];
#pragma unroll
                    for (int i = 0; i < VEC; ++i) part[t].v[i] = part[t].v[i] + o.v[i];
                }
            T *crow = a.carry + (int64_t)seg * a.F;
#pragma unroll
            for (int t = 0; t < TILES; ++t)
                if (foff[t] >= 0) store_pack<T, VEC>(crow + foff[t], part[t]);
        }
    }
    if (lane == 0 && blockIdx.y == 0) a.carry_row[seg] = mark;
}

// One level of the carry reduction.  Carries (row, vector) with equal rows are adjacent
// (in the list the nnz kernel writes, kMerged entries may lie between them: they are
// skipped); kNoCarry marks a run that carries nothing.  A lane group takes kCarryFan
// consecutive carries:
// a row whose carries all lie inside the chunk is finished here (Y += their sum, nobody
// else touches that row); the part of a row that reaches the chunk from before goes to
// slot 2*chunk of the next level, the part of a row that goes on behind the chunk to slot
// 2*chunk+1 (a row that covers the whole chunk fills slot 2*chunk and puts zeros in the
// other), so that equal rows are adjacent again on the next level.
constexpr int kCarryFan = 64;
constexpr int kReduceBatch = 16;  // carry rows in flight per lane group
constexpr int kFixBatch = 8;

template <typename T, int VEC, int LPR>
__global__ __launch_bounds__(kBlock) void spmm_carry_reduce_kernel(SpmmArgs<T> a) {
    constexpr int GPB = kBlock / LPR;
    const int sub = threadIdx.x % LPR;
    const int chunk = blockIdx.x * GPB + threadIdx.x / LPR;
    const int s0 = chunk * kCarryFan;
    if (s0 >= a.nseg) return;
    const int s1 = min(s0 + kCarryFan, a.nseg);
    const bool merged = a.merge_stride > 1;  // the list of the nnz kernel: s0 starts a workgroup
    const int before = (s0 > 0 && !merged) ? a.carry_row[s0 - 1] : -1;
    const int after = s1 < a.nseg ? a.carry_row[s1] : -1;
    // the rows of the chunk: every lane of the group reads all of them (same addresses,
    // one round trip), so no lane has to wait for another
    int rr[kCarryFan];
    if (s1 - s0 == kCarryFan) {
        const int4 *p = reinterpret_cast<const int4 *>(a.carry_row + s0);  // s0 is a multiple of 64
#pragma unroll
        for (int q = 0; q < kCarryFan / 4; ++q) {
            const int4 v = p[q];
            rr[4 * q] = v.x, rr[4 * q + 1] = v.y, rr[4 * q + 2] = v.z, rr[4 * q + 3] = v.w;
        }
    } else {
#pragma unroll
        for (int u = 0; u < kCarryFan; ++u) rr[u] = s0 + u < s1 ? a.carry_row[s0 + u] : -1;
    }
    int any = -1;
#pragma unroll
    for (int u = 0; u < kCarryFan; ++u) any = max(any, rr[u]);
    if (any < 0) {  // nothing is carried through this chunk
        if (sub == 0) a.carry_row_out[2 * chunk] = a.carry_row_out[2 * chunk + 1] = -1;
        return;
    }
    int head_row = -1, tail_row = -1;
    T *slot0 = a.carry_out + (int64_t)(2 * chunk) * a.F;
    T *slot1 = slot0 + a.F;
    for (int64_t f = (int64_t)sub * VEC; f < a.F; f += (int64_t)LPR * VEC) {
        Pack<T, VEC> acc, zero;
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc.v[i] = zero.v[i] = T(0);
        int cur = -1;
        bool from_before = false;
        auto close = [&](bool ends_here) {
            if (cur < 0) return;
            if (!from_before && ends_here) {
                // The one addition to these elements in this launch sequence (the row's
                // last run has stored its part already), so its result does not depend on
                // timing; sent as an atomic only so that the lane need not wait for Y.
                T *y = a.Y + (int64_t)out_row(a, cur) * a.F + f;
#pragma unroll
                for (int i = 0; i < VEC; ++i) unsafeAtomicAdd(y + i, acc.v[i]);
                return;
            }
            if (from_before) {
                head_row = cur;
                store_pack<T, VEC>(slot0 + f, acc);
                if (!ends_here) {
                    tail_row = cur;
                    store_pack<T, VEC>(slot1 + f, zero);
                }
            } else {
                tail_row = cur;
                store_pack<T, VEC>(slot1 + f, acc);
            }
        };
#pragma unroll
        for (int b = 0; b < kCarryFan; b += kReduceBatch) {
            Pack<T, VEC> c[kReduceBatch];
#pragma unroll
            for (int u = 0; u < kReduceBatch; ++u)
                c[u] = rr[b + u] >= 0 ? load_pack<T, VEC>(a.carry + (int64_t)(s0 + b + u) * a.F + f) : zero;
#pragma unroll
            for (int u = 0; u < kReduceBatch; ++u) {
                if (rr[b + u] != cur && rr[b + u] != kMerged) {  // entries behind the end of the last chunk are -1
                    close(true);
                    cur = rr[b + u];
                    acc = zero;
                    // is the row carried into the chunk?  In the list of the nnz kernel the
                    // run before s0 may be a merged one, so ask where the row starts.
                    from_before = (b + u == 0) && cur >= 0 &&
                                  (merged ? (int64_t)a.rowptr[cur] < (int64_t)s0 * a.seg_nnz : cur == before);
                }
#pragma unroll
                for (int i = 0; i < VEC; ++i) acc.v[i] = acc.v[i] + c[u].v[i];
            }
        }
        close(!(cur >= 0 && cur == after));
    }
    if (sub == 0) {
        a.carry_row_out[2 * chunk] = head_row;
        a.carry_row_out[2 * chunk + 1] = tail_row;
    }
}

// Adds the carries of every row that straddles runs, in ascending run order, and
// (when not accumulating) clears the rows that have no entries (the two sets of rows are
// disjoint).  Carries: one lane group (LPR lanes across the features) per run; the group
// whose run holds the first carry of a row walks the row's carries, kFixBatch in flight,
// and adds their sum to the row.  Empty rows: one thread looks at one row, and the empty
// rows of a wave are then dealt out to its lane groups.

// Lane (within the wave) of the flagged item this lane's group should handle in the
// round that starts at rank `base`, or -1.  Uniform control flow: every lane calls it.
template <int LPR>
__device__ __forceinline__ int deal_item(bool flag, int my_rank, int base, int grp) {
    constexpr int G = kWave / LPR;
    int src = -1;
#pragma unroll
    for (int gi = 0; gi < G; ++gi) {
        const unsigned long long m = __ballot(flag && my_rank == base + gi);
        if (gi == grp && m) src = __ffsll(m) - 1;
    }
    return src;
}

template <typename T, int VEC, int LPR, bool MERGED>
__global__ __launch_bounds__(kBlock) void spmm_fixup_kernel(SpmmArgs<T> a) {
    constexpr int GPB = kBlock / LPR;
    // carry rows in flight per lane group; few, so that the many groups that find nothing
    // to do are all resident at once
    constexpr int BATCH = MERGED ? 4 : kFixBatch;
    const int lane = threadIdx.x % kWave;
    const int sub = lane % LPR, grp = lane / LPR;

    int s0 = blockIdx.x * GPB + threadIdx.x / LPR;
    if constexpr (LPR == kWave) s0 = __builtin_amdgcn_readfirstlane(s0);
    const int stride = MERGED ? a.merge_stride : 1;  // MERGED: the list of the nnz kernel
    // First carry of its row?  The list of the nnz kernel holds one carry per row and
    // workgroup: a row has an earlier carry exactly when it starts before this run, and
    // its later carries belong to the first run of every following workgroup whose end
    // still lies inside the row.  In a plain list the carries of a row are adjacent.
    int row = -1, row_end = 0;
    if (s0 < a.nseg) {
        const int r = a.carry_row[s0];
        if (r >= 0) {
            bool head;
            if constexpr (MERGED) {
                head = (int64_t)a.rowptr[r] >= (int64_t)s0 * a.seg_nnz;
                row_end = a.rowptr[r + 1];
            } else {
                head = s0 == 0 || a.carry_row[s0 - 1] != r;
            }
            if (head) row = r;
        }
    }
    if (row >= 0) {
        const int64_t group0 = (int64_t)(s0 / stride) * stride;
#pragma unroll 1
        for (int64_t f = (int64_t)sub * VEC; f < a.F; f += (int64_t)LPR * VEC) {
            Pack<T, VEC> acc, zero;
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc.v[i] = zero.v[i] = T(0);
            bool more = true;
#pragma unroll 1
            for (int k = 0; more; k += BATCH) {
                bool take[BATCH];
                Pack<T, VEC> c[BATCH];
                if constexpr (MERGED) {
#pragma unroll
                    for (int u = 0; u < BATCH; ++u) {
                        const int64_t p = (k + u == 0) ? (int64_t)s0 : group0 + (int64_t)(k + u) * stride;
                        take[u] = (k + u == 0) || (p + 1) * a.seg_nnz < (int64_t)row_end;
                        c[u] = take[u] ? load_pack<T, VEC>(a.carry + p * a.F + f) : zero;
                    }
                } else {
                    int rr[BATCH];
#pragma unroll
                    for (int u = 0; u < BATCH; ++u) {
                        const int64_t p = (int64_t)s0 + k + u;
                        take[u] = p < a.nseg;
                        const int64_t idx = take[u] ? p : (int64_t)a.nseg - 1;
                        rr[u] = a.carry_row[idx];
                        c[u] = load_pack<T, VEC>(a.carry + idx * a.F + f);
                    }
#pragma unroll
                    for (int u = 0; u < BATCH; ++u) take[u] = take[u] && rr[u] == row;
                }
#pragma unroll
                for (int u = 0; u < BATCH; ++u) {
                    more = more && take[u];
                    if (more)
#pragma unroll
                        for (int i = 0; i < VEC; ++i) acc.v[i] = acc.v[i] + c[u].v[i];
                }
            }
            T *y = a.Y + (int64_t)out_row(a, row) * a.F + f;
            Pack<T, VEC> o = load_pack<T, VEC>(y);
#pragma unroll
            for (int i = 0; i < VEC; ++i) o.v[i] = o.v[i] + acc.v[i];
            store_pack<T, VEC>(y, o);
        }
    }

    if (a.accumulate) return;
    const int item = blockIdx.x * kBlock + threadIdx.x;
    const int wave_item0 = item - lane;
    if (wave_item0 >= a.rows) return;
    const bool empty = item < a.rows && a.rowptr[item] == a.rowptr[item + 1];
    const unsigned long long below = (1ull << lane) - 1ull;
    const unsigned long long empties = __ballot(empty);
    const int n_empty = __popcll(empties), empty_rank = __popcll(empties & below);
    constexpr int G = kWave / LPR;
    for (int base = 0; base < n_empty; base += G) {
        const int src = deal_item<LPR>(empty, empty_rank, base, grp);
        if (src < 0) continue;
        const int erow = out_row(a, wave_item0 + src);
        Pack<T, VEC> zero;
#pragma unroll
        for (int i = 0; i < VEC; ++i) zero.v[i] = T(0);
        for (int64_t f = (int64_t)sub * VEC; f < a.F; f += (int64_t)LPR * VEC)
            store_pack_stream<T, VEC>(a.Y + (int64_t)erow * a.F + f, zero);
    }
}

// The same pass for a block that comes with the lists of its cut rows and its empty rows
// (both follow from rowptr and the run length alone, so they are made once per block): a lane
// group per cut row, and nothing for the many runs that carry nothing.  The carries of a row
// sit where the nnz kernel's workgroups left them: at the run the row starts in, and at the first
// run of every following workgroup whose end still lies inside the row; they are added in that
// (ascending) order, the same as in spmm_fixup_kernel, so the result is the same bit for bit.
template <typename T, int VEC, int LPR>
__global__ __launch_bounds__(kBlock) void spmm_fixup_rows_kernel(SpmmArgs<T> a) {
    constexpr int GPB = kBlock / LPR;
    constexpr int BATCH = 8;
    const int sub = threadIdx.x % LPR;
    int item = blockIdx.x * GPB + threadIdx.x / LPR;
    if constexpr (LPR == kWave) item = __builtin_amdgcn_readfirstlane(item);
    if (item < a.n_cut_rows) {
        const int row = a.cut_rows[item];
        const int64_t row_end = a.rowptr[row + 1];
        const int64_t s0 = a.rowptr[row] / a.seg_nnz;           // the run the row starts in
        const int64_t group0 = s0 / a.merge_stride * a.merge_stride;  // first run of that run's workgroup
#pragma unroll 1
        for (int64_t f = (int64_t)sub * VEC; f < a.F; f += (int64_t)LPR * VEC) {
            Pack<T, VEC> acc, zero;
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc.v[i] = zero.v[i] = T(0);
            bool more = true;
#pragma unroll 1
            for (int k = 0; more; k += BATCH) {
                bool take[BATCH];
                Pack<T, VEC> c[BATCH];
#pragma unroll
                for (int u = 0; u < BATCH; ++u) {
                    const int64_t p = (k + u == 0) ? s0 : group0 + (int64_t)(k + u) * a.merge_stride;
                    take[u] = (k + u == 0) || (p + 1) * a.seg_nnz < row_end;
                    c[u] = take[u] ? load_pack<T, VEC>(a.carry + p * a.F + f) : zero;
                }
#pragma unroll
                for (int u = 0; u < BATCH; ++u) {
                    more = more && take[u];
                    if (more)
#pragma unroll
                        for (int i = 0; i < VEC; ++i) acc.v[i] = acc.v[i] + c[u].v[i];
                }
            }
            T *y = a.Y + (int64_t)out_row(a, row) * a.F + f;
            Pack<T, VEC> o = load_pack<T, VEC>(y);
#pragma unroll
            for (int i = 0; i < VEC; ++i) o.v[i] = o.v[i] + acc.v[i];
            store_pack<T, VEC>(y, o);
        }
    }
    if (a.accumulate || item >= a.n_empty_rows) return;
    const int erow = out_row(a, a.empty_rows[item]);
    Pack<T, VEC> zero;
#pragma unroll
    for (int i = 0; i < VEC; ++i) zero.v[i] = T(0);
    for (int64_t f = (int64_t)sub * VEC; f < a.F; f += (int64_t)LPR * VEC)
        store_pack_stream<T, VEC>(a.Y + (int64_t)erow * a.F + f, zero);
}

// ------------------------------------------------------------------- dispatch --
struct Shape {
    int vec, lpr, tiles, grid_y;
};

// Lane layout for a feature width: the widest vector the width and the pointers'
// alignment allow, then as many lanes as a row needs (power of two, 4..64).
// min_lpr: narrow the vectors (down to single words) while a row would take fewer lanes than
// this.  The nnz schedule asks for 16: with 4 lanes per run a wave walks 16 runs at once, each
// with its own row changes (F = 16: 0.106 -> 0.089 ms for the forward vertex stage of the web
// graph); the row schedule is faster with the widest vectors (0.036 against 0.053 ms).
template <typename T>
Shape pick_shape(int64_t F, const void *p0, const void *p1, const void *p2, const void *p3, int min_lpr = 4) {
    auto aligned = [&](size_t bytes) {
        auto ok = [&](const void *p) { return p == nullptr || (reinterpret_cast<uintptr_t>(p) % bytes) == 0; };
        return ok(p0) && ok(p1) && ok(p2) && ok(p3);
    };
    Shape s;
    s.vec = 1;
    if (sizeof(T) == 4) {
        if (F % 4 == 0 && aligned(16)) s.vec = 4;
        else if (F % 2 == 0 && aligned(8)) s.vec = 2;
        while (s.vec > 1 && F / s.vec < min_lpr) s.vec /= 2;
    }
    const int64_t slots = F / s.vec;
    int lpr = pow2_ceil(slots);
    if (lpr < 4) lpr = 4;
    if (lpr > 64) lpr = 64;
    if (s.vec != 4 || sizeof(T) != 4) {
        // fewer instantiations off the main path: 4, 16 or 64 lanes per row
        lpr = lpr <= 4 ? 4 : (lpr <= 16 ? 16 : 64);
    }
    s.lpr = lpr;
    s.tiles = (lpr == 64 && slots > 64 && sizeof(T) == 4) ? 2 : 1;
    s.grid_y = (int)ceil_div(slots, (int64_t)s.lpr * s.tiles);
    return s;
}

enum { KIND_ROW = 0, KIND_NNZ = 1, KIND_FIXUP = 2, KIND_REDUCE = 3, KIND_FIXUP_ROWS = 4 };

template <typename T, int VEC, int LPR, int TILES>
int launch_shape(int kind, int mode, const SpmmArgs<T> &args, int64_t items, int grid_y, hipStream_t stream) {
    constexpr int GPB = kBlock / LPR;
    dim3 grid((unsigned)ceil_div(items, GPB), (unsigned)grid_y), block(kBlock);
    if (grid.x == 0) return CGNN_OK;
    SpmmArgs<T> a = args;
    a.stretch_log2 = 0;
    if (kind == KIND_ROW || kind == KIND_NNZ) {
        a.stretch_log2 = stretch_log2_for<GPB>(grid.x);
        a.blocks = (int32_t)grid.x;
        grid.x = (unsigned)(ceil_div((int64_t)grid.x, kXcds) * kXcds);
    }
    switch (kind) {
        case KIND_ROW:
            if (mode == MODE_DUAL)
                hipLaunchKernelGGL((spmm_row_kernel<T, VEC, LPR, TILES, MODE_DUAL>), grid, block, 0, stream, a);
            else
                hipLaunchKernelGGL((spmm_row_kernel<T, VEC, LPR, TILES, MODE_VAL>), grid, block, 0, stream, a);
            break;
        case KIND_NNZ:
            if (mode == MODE_VAL)
                hipLaunchKernelGGL((spmm_nnz_kernel<T, VEC, LPR, TILES, MODE_VAL>), grid, block, 0, stream, a);
            else if (mode == MODE_UNIT)
                hipLaunchKernelGGL((spmm_nnz_kernel<T, VEC, LPR, TILES, MODE_UNIT>), grid, block, 0, stream, a);
            else if (mode == MODE_DUAL)
                hipLaunchKernelGGL((spmm_nnz_kernel<T, VEC, LPR, TILES, MODE_DUAL>), grid, block, 0, stream, a);
            else if (mode == MODE_SIGN_MASK)
                hipLaunchKernelGGL((spmm_nnz_kernel<T, VEC, LPR, TILES, MODE_SIGN_MASK>), grid, block, 0, stream, a);
            else
                hipLaunchKernelGGL((spmm_nnz_kernel<T, VEC, LPR, TILES, MODE_RELU_MASK>), grid, block, 0, stream, a);
            break;
        case KIND_FIXUP: {  // a lane group per carry, and (when not accumulating) a thread per row
            const int64_t for_rows = a.accumulate ? 0 : ceil_div((int64_t)a.rows, kBlock);
            const int64_t for_carries = ceil_div((int64_t)a.nseg, GPB);
            const dim3 fix_grid((unsigned)(for_rows > for_carries ? for_rows : for_carries));
            if (fix_grid.x > 0 && a.merge_stride > 1)
                hipLaunchKernelGGL((spmm_fixup_kernel<T, VEC, LPR, true>), fix_grid, block, 0, stream, a);
            else if (fix_grid.x > 0)  // the short list a reduction level leaves
                hipLaunchKernelGGL((spmm_fixup_kernel<T, VEC, LPR, false>), fix_grid, block, 0, stream, a);
            break;
        }
        case KIND_FIXUP_ROWS:  // items = lane groups: one per cut row, one per empty row
            hipLaunchKernelGGL((spmm_fixup_rows_kernel<T, VEC, LPR>), dim3((unsigned)ceil_div(items, GPB)), block, 0, stream,
                               a);
            break;
        case KIND_REDUCE:  // items = chunks of kCarryFan carries, one lane group each
            hipLaunchKernelGGL((spmm_carry_reduce_kernel<T, VEC, LPR>), dim3((unsigned)ceil_div(items, GPB)), block, 0,
                               stream, a);
            break;
    }
    return check_launch("spmm launch");
}

#define CGNN_SHAPE_CASE(V, L, TL)                   \
    if (s.vec == V && s.lpr == L && s.tiles == TL)  \
        return launch_shape<T, V, L, TL>(kind, mode, a, items, s.grid_y, stream);

template <typename T>
int launch(int kind, int mode, const Shape &s, const SpmmArgs<T> &a, int64_t items, hipStream_t stream) {
    if constexpr (sizeof(T) == 4) {
        CGNN_SHAPE_CASE(4, 4, 1)
        CGNN_SHAPE_CASE(4, 8, 1)
        CGNN_SHAPE_CASE(4, 16, 1)
        CGNN_SHAPE_CASE(4, 32, 1)
        CGNN_SHAPE_CASE(4, 64, 1)
        CGNN_SHAPE_CASE(4, 64, 2)
        CGNN_SHAPE_CASE(2, 4, 1)
        CGNN_SHAPE_CASE(2, 16, 1)
        CGNN_SHAPE_CASE(2, 64, 1)
        CGNN_SHAPE_CASE(2, 64, 2)
        CGNN_SHAPE_CASE(1, 4, 1)
        CGNN_SHAPE_CASE(1, 16, 1)
        CGNN_SHAPE_CASE(1, 64, 1)
        CGNN_SHAPE_CASE(1, 64, 2)
    } else {
        CGNN_SHAPE_CASE(1, 4, 1)
        CGNN_SHAPE_CASE(1, 16, 1)
        CGNN_SHAPE_CASE(1, 64, 1)
    }
    return fail(CGNN_EUNSUPPORTED, "spmm: no kernel for this lane layout");
}

// AUTO: rows are "near regular" when the longest one is a small multiple of the mean;
// otherwise balance by non-zeros.
int schedule_for(int64_t rows, int64_t nnz, int32_t max_row_nnz, int kernel) {
    if (kernel == CGNN_SPMM_ROW || kernel == CGNN_SPMM_NNZ) return kernel;
    if (max_row_nnz <= 0) return CGNN_SPMM_NNZ;
    const double mean = rows > 0 ? (double)nnz / (double)rows : 0.0;
    const double limit = 8.0 * (mean < 8.0 ? 8.0 : mean);
    return (double)max_row_nnz <= limit ? CGNN_SPMM_ROW : CGNN_SPMM_NNZ;
}

int resolve_kernel(const cgnn_csr *A, int kernel) {
    if (kernel == CGNN_SPMM_ROW || kernel == CGNN_SPMM_NNZ) return kernel;
    if (A->rowidx == nullptr) return CGNN_SPMM_ROW;  // the nnz schedule needs the row of every non-zero
    return schedule_for(A->rows, A->nnz, A->max_row_nnz, kernel);
}

int seg_len(const cgnn_csr *A) {
    int s = A->seg_nnz > 0 ? A->seg_nnz : kDefaultSeg;
    return (s + kUnroll - 1) / kUnroll * kUnroll;
}

int check_csr(const cgnn_csr *A, const char *name) {
    if (A == nullptr) return fail(CGNN_EINVAL, "spmm: null csr");
    const int64_t lim = (int64_t)INT32_MAX - 65536;  // room for run ends past the last entry
    if (A->rows < 0 || A->cols < 0 || A->nnz < 0 || A->rows >= lim || A->nnz >= lim || A->cols >= lim) {
        set_error("%s: rows/cols/nnz must be in [0, 2^31 - 65536)", name);
        return CGNN_EINVAL;
    }
    if (A->rowptr == nullptr || (A->nnz > 0 && A->colidx == nullptr)) {
        set_error("%s: rowptr/colidx must not be null", name);
        return CGNN_EINVAL;
    }
    return CGNN_OK;
}

template <typename T>
SpmmArgs<T> make_args(const cgnn_csr *A, const void *X, const void *X1, int64_t split, const void *M, void *Y,
                      int64_t F, int accumulate) {
    SpmmArgs<T> a{};
    a.rowptr = A->rowptr;
    a.colidx = A->colidx;
    a.rowidx = A->rowidx;
    a.rowmap = A->rowmap;
    a.val = static_cast<const T *>(A->val);
    a.X = static_cast<const T *>(X);
    a.X1 = static_cast<const T *>(X1);
    a.M = static_cast<const T *>(M);
    a.Y = static_cast<T *>(Y);
    a.F = F;
    a.rows = (int32_t)A->rows;
    a.nnz = (int32_t)A->nnz;
    a.split = (int32_t)split;
    a.accumulate = accumulate ? 1 : 0;
    return a;
}

// Workspace of the nnz schedule: per level the rows of the carries, then the carries.
// Level 0 has one carry per run; every further level has two per kCarryFan carries of the
// one before; levels are added until at most kSerialCarries carries are left.
constexpr int64_t kSerialCarries = 256;
constexpr int kMaxCarryLevels = 8;

struct CarryLevels {
    int count = 0;
    int64_t n[kMaxCarryLevels];
    size_t row_off[kMaxCarryLevels], carry_off[kMaxCarryLevels];
    size_t total = 0;
};

// Rows whose carries the fix-up pass can walk directly (at most kLongChain of them, one per
// workgroup of the nnz kernel) need no reduction levels.  max_row_nnz == 0 means unknown.
constexpr int64_t kLongChain = 256;

bool wants_levels(const cgnn_csr *A, int seg, int runs_per_workgroup) {
    return A->max_row_nnz <= 0 || (int64_t)A->max_row_nnz > kLongChain * seg * runs_per_workgroup;
}

CarryLevels carry_levels(int64_t nseg, int64_t F, size_t elt, bool reduce) {
    CarryLevels L;
    int64_t n = nseg;
    while (n > 0) {
        const int k = L.count++;
        L.n[k] = n;
        L.row_off[k] = L.total;
        L.total += align_up((size_t)n * sizeof(int32_t), 256);
        L.carry_off[k] = L.total;
        L.total += align_up((size_t)n * (size_t)F * elt, 256);
        if (!reduce || n <= kSerialCarries || L.count == kMaxCarryLevels) break;
        n = 2 * ceil_div(n, kCarryFan);
    }
    return L;
}

template <typename T>
int spmm_typed(const cgnn_csr *A, const void *X, const void *X1, int64_t split, const void *M, void *Y, int64_t F,
               int accumulate, int kernel, int mode, void *ws, size_t ws_bytes, hipStream_t stream) {
    if (A->rows == 0 || F == 0) return CGNN_OK;
    if (mode != MODE_DUAL) split = INT32_MAX;  // every column comes from X
    SpmmArgs<T> a = make_args<T>(A, X, X1, split, M, Y, F, accumulate);
    const bool masked = mode == MODE_RELU_MASK || mode == MODE_SIGN_MASK;
    a.read_once = mode == MODE_UNIT || masked;  // asked for by name: the cluster reductions
    if (mode == MODE_SIGN_MASK) {  // M holds bits, not rows
        a.signs = static_cast<const uint32_t *>(M);
        a.sign_words = (int32_t)ceil_div(F, 32);
        a.M = nullptr;
        M = nullptr;
    }
    kernel = resolve_kernel(A, kernel);
    if (masked) kernel = CGNN_SPMM_NNZ;  // masks exist for the nnz schedule only
    // unit values without the multiplications; a product that adds to Y stays with the plain mode, the only one that reads Y
    if (mode == MODE_VAL && A->val == nullptr && kernel == CGNN_SPMM_NNZ && !accumulate) mode = MODE_UNIT;
    if (mode == MODE_DUAL && A->nnz > 0 && A->val == nullptr)
        return fail(CGNN_EINVAL, "spmm: the two-source product needs stored values");
    if (kernel == CGNN_SPMM_ROW) {
        Shape s = pick_shape<T>(F, X, Y, X1, nullptr);
        return launch<T>(KIND_ROW, mode, s, a, A->rows, stream);
    }
    if (A->nnz > 0 && A->rowidx == nullptr) return fail(CGNN_EINVAL, "spmm: nnz schedule needs rowidx");
    const int seg = seg_len(A);
    const int64_t nseg = ceil_div(A->nnz, seg);
    // the lane layout decides how many runs a workgroup merges (the carries sit at multiples
    // of 256 bytes in the workspace, so the workspace stands for them in the alignment check)
    const Shape s = pick_shape<T>(F, X, Y, ws, mode == MODE_DUAL ? X1 : M, 16);
    const int runs_per_workgroup = kBlock / s.lpr;
    const CarryLevels levels = carry_levels(nseg, F, sizeof(T), wants_levels(A, seg, runs_per_workgroup));
    if (nseg > 0 && (ws == nullptr || ws_bytes < levels.total)) {
        set_error("spmm: workspace of %zu bytes needed, %zu given", levels.total, ws_bytes);
        return CGNN_EWORKSPACE;
    }
    char *base = static_cast<char *>(ws);
    auto level_rows = [&](int k) { return reinterpret_cast<int32_t *>(base + levels.row_off[k]); };
    auto level_carries = [&](int k) { return reinterpret_cast<T *>(base + levels.carry_off[k]); };
    a.nseg = (int32_t)nseg;
    a.seg_nnz = seg;
    a.run_start = A->run_start;
    a.carry_row = nseg > 0 ? level_rows(0) : nullptr;
    a.carry = nseg > 0 ? level_carries(0) : nullptr;
    a.merge_stride = runs_per_workgroup;
    if (nseg > 0) {
        int rc = launch<T>(KIND_NNZ, mode, s, a, nseg, stream);
        if (rc != CGNN_OK) return rc;
    }
    for (int k = 0; k + 1 < levels.count; ++k) {
        a.nseg = (int32_t)levels.n[k];
        a.carry_row = level_rows(k);
        a.carry = level_carries(k);
        a.carry_row_out = level_rows(k + 1);
        a.carry_out = level_carries(k + 1);
        a.merge_stride = k == 0 ? runs_per_workgroup : 1;
        int rc = launch<T>(KIND_REDUCE, mode, s, a, ceil_div(levels.n[k], kCarryFan), stream);
        if (rc != CGNN_OK) return rc;
    }
    if (levels.count > 0) {
        const int last = levels.count - 1;
        a.nseg = (int32_t)levels.n[last];
        a.carry_row = level_rows(last);
        a.carry = level_carries(last);
        a.merge_stride = last == 0 ? runs_per_workgroup : 1;
    }
    if (A->cut_rows != nullptr && levels.count == 1) {
        // the block knows which rows its runs cut (and which rows are empty): only those are looked at
        a.cut_rows = A->cut_rows;
        a.n_cut_rows = A->n_cut_rows;
        a.empty_rows = A->empty_rows;
        a.n_empty_rows = accumulate ? 0 : A->n_empty_rows;
        const int64_t items = a.n_cut_rows > a.n_empty_rows ? a.n_cut_rows : a.n_empty_rows;
        return launch<T>(KIND_FIXUP_ROWS, mode, s, a, items, stream);
    }
    const int64_t items = accumulate ? a.nseg : (a.nseg > A->rows ? a.nseg : A->rows);
    return launch<T>(KIND_FIXUP, mode, s, a, items, stream);
}

// ------------------------------------------------------- CSR preparation -------

__global__ void narrow_i64_kernel(const int64_t *__restrict__ src, int32_t *__restrict__ dst, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
         i += (int64_t)gridDim.x * blockDim.x)
        dst[i] = (int32_t)src[i];
}

// run_start[s] = where the run of the nnz schedule that covers position s * seg begins.
__global__ void run_starts_kernel(const int32_t *__restrict__ rowptr, const int32_t *__restrict__ rowidx, int32_t nnz,
                                  int32_t seg, int64_t n, int32_t *__restrict__ run_start) {
    const int64_t s = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (s >= n) return;
    const int64_t e = s * seg;
    if (e >= nnz) {
        run_start[s] = nnz;
        return;
    }
    const int r = rowidx[e];
    const int s0 = rowptr[r];
    run_start[s] = (rowptr[r + 1] - s0 <= seg) ? s0 : (int32_t)e;
}

// rowidx[e] = largest r with rowptr[r] <= e (rows without entries are skipped).
template <typename P>
__global__ void expand_rows_kernel(const P *__restrict__ rowptr, int64_t rows, int64_t nnz,
                                   int32_t *__restrict__ rowidx) {
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < nnz;
         e += (int64_t)gridDim.x * blockDim.x) {
        int64_t lo = 0, hi = rows;  // invariant: rowptr[lo] <= e < rowptr[hi]
        while (hi - lo > 1) {
            int64_t mid = (lo + hi) >> 1;
            if ((int64_t)rowptr[mid] <= e) lo = mid;
            else hi = mid;
        }
        rowidx[e] = (int32_t)lo;
    }
}

unsigned grid_for(int64_t n) {
    int64_t b = ceil_div(n, kBlock);
    return (unsigned)(b > 16384 ? 16384 : b);
}

// narrow[c] = ids[c] as int32 (an id outside [0, groups) is replaced by the nearest valid one and
// reported): the table the composition below gathers from, half the size of the int64 ids.
__global__ void narrow_ids_kernel(const int64_t *__restrict__ ids, int64_t n, int64_t groups, int32_t *__restrict__ narrow,
                                  int32_t *__restrict__ bad) {
    for (int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; c < n; c += (int64_t)gridDim.x * blockDim.x) {
        int64_t id = ids[c];
        if (id < 0 || id >= groups) {
            if (bad) *bad = 1;  // every writer stores the same value
            id = id < 0 ? 0 : groups - 1;
        }
        narrow[c] = (int32_t)id;
    }
}

// out[e] = narrow[col[e]] for the columns below first_cols, the other columns unchanged.  Four
// entries per thread, their table reads in flight together.
__global__ void compose_columns_kernel(const int32_t *__restrict__ col, int64_t nnz, int64_t first_cols,
                                       const int32_t *__restrict__ narrow, int32_t *__restrict__ out) {
    const int64_t quads = nnz / 4;
    for (int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; q < quads; q += (int64_t)gridDim.x * blockDim.x) {
        const int4 c = reinterpret_cast<const int4 *>(col)[q];
        int4 r;
        r.x = c.x < first_cols ? narrow[c.x] : c.x;
        r.y = c.y < first_cols ? narrow[c.y] : c.y;
        r.z = c.z < first_cols ? narrow[c.z] : c.z;
        r.w = c.w < first_cols ? narrow[c.w] : c.w;
        reinterpret_cast<int4 *>(out)[q] = r;
    }
    const int64_t e = quads * 4 + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e < nnz) {
        const int32_t c = col[e];
        out[e] = c < first_cols ? narrow[c] : c;
    }
}

}  // namespace

// Entry used by the cluster reductions (unit values; mask: 0 none, 1 the rows of M, where M <= 0 drops
// the element, 2 M holds ceil(F / 32) words of bits per row, where a clear bit drops it).
int spmm_members(const cgnn_csr *A, int dtype, const void *X, const void *M, void *Y, int64_t F,
                 int mask, void *ws, size_t ws_bytes, hipStream_t stream) {
    const int mode = mask == 2 ? MODE_SIGN_MASK : (mask == 1 ? MODE_RELU_MASK : MODE_UNIT);
    if (dtype == CGNN_F32)
        return spmm_typed<float>(A, X, nullptr, 0, M, Y, F, 0, CGNN_SPMM_NNZ, mode, ws, ws_bytes, stream);
    if (dtype == CGNN_F64)
        return spmm_typed<double>(A, X, nullptr, 0, M, Y, F, 0, CGNN_SPMM_NNZ, mode, ws, ws_bytes, stream);
    return fail(CGNN_EUNSUPPORTED, "spmm: dtype must be f32 or f64");
}

// ------------------------------------------- scratch that nobody allocates -------
//
// cgnn_spmm_static runs the same kernels as cgnn_spmm with the carries of the nnz schedule in
// an array that is part of the library's device image, for callers that cannot allocate.
// Every GPU the library runs on holds its own copy of the array, at its own address, from the
// moment the image is loaded there until the process ends.
constexpr size_t kStaticScratchBytes = size_t(64) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

constexpr int kMaxDevices = 64;
std::mutex static_scratch_lock;
void *static_scratch_of_device[kMaxDevices] = {};

// The address of `scratch` on the device that is current in the calling thread.  In host code
// the name `scratch` is only a handle for the symbol: the device address comes from
// hipGetSymbolAddress, once per device, and is what kernels and copies are given.
int static_scratch(void **out) {
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess || device < 0 || device >= kMaxDevices) {
        set_error("cgnn_spmm_static: no usable current device (%s)", e != hipSuccess ? hipGetErrorString(e) : "index out of range");
        return CGNN_ELAUNCH;
    }
    std::lock_guard<std::mutex> hold(static_scratch_lock);
    if (static_scratch_of_device[device] == nullptr) {
        void *ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr) {
            set_error("cgnn_spmm_static: hipGetSymbolAddress failed on device %d: %s", device, hipGetErrorString(e));
            return CGNN_ELAUNCH;
        }
        static_scratch_of_device[device] = ptr;
    }
    *out = static_scratch_of_device[device];
    return CGNN_OK;
}

}  // namespace

}  // namespace cgnn

using namespace cgnn;

extern "C" int cgnn_spmm_schedule(int64_t rows, int64_t nnz, int32_t max_row_nnz, int kernel) {
    if (kernel < CGNN_SPMM_AUTO || kernel > CGNN_SPMM_NNZ) return CGNN_SPMM_AUTO;
    return schedule_for(rows, nnz, max_row_nnz, kernel);
}

extern "C" int cgnn_spmm_run_length(const cgnn_csr *A) { return A == nullptr ? 0 : seg_len(A); }

extern "C" size_t cgnn_spmm_static_scratch_bytes(void) { return kStaticScratchBytes; }

extern "C" int cgnn_spmm_static_init(void) {
    void *ws = nullptr;
    return static_scratch(&ws);
}

extern "C" int cgnn_spmm_static(const cgnn_csr *A, int dtype, const void *X, void *Y, int64_t F, int accumulate,
                                int kernel, cgnn_stream_t stream) {
    int rc = check_csr(A, "cgnn_spmm_static");
    if (rc != CGNN_OK) return rc;
    CGNN_REQUIRE(F >= 0, "cgnn_spmm_static: F must be non-negative");
    CGNN_REQUIRE(kernel >= CGNN_SPMM_AUTO && kernel <= CGNN_SPMM_NNZ, "cgnn_spmm_static: unknown kernel id");
    CGNN_REQUIRE(dtype == CGNN_F32 || dtype == CGNN_F64, "cgnn_spmm_static: dtype must be f32 or f64");
    const size_t need = cgnn_spmm_workspace_bytes(A, F, dtype, kernel);
    if (need > kStaticScratchBytes) {
        set_error("cgnn_spmm_static: this product needs %zu bytes of scratch, the built-in array holds %zu; use "
                  "cgnn_spmm with a workspace of the caller's",
                  need, kStaticScratchBytes);
        return CGNN_EWORKSPACE;
    }
    void *ws = nullptr;
    if (need > 0) {
        rc = static_scratch(&ws);
        if (rc != CGNN_OK) return rc;
    }
    // The kernels write every carry slot and every carry-row entry they later read, so the
    // contents a previous call left in the array need no clearing.
    return cgnn_spmm(A, dtype, X, Y, F, accumulate, kernel, ws, need > 0 ? kStaticScratchBytes : 0, stream);
}

extern "C" size_t cgnn_spmm_workspace_bytes(const cgnn_csr *A, int64_t F, int dtype, int kernel) {
    if (A == nullptr || A->nnz <= 0 || F <= 0) return 0;
    if (resolve_kernel(A, kernel) == CGNN_SPMM_ROW) return 0;
    const int seg = seg_len(A);
    // an upper bound: the lane layout (which depends on the pointers' alignment) can only
    // remove reduction levels
    return carry_levels(ceil_div(A->nnz, seg), F, dtype == CGNN_F64 ? 8 : 4, wants_levels(A, seg, 1)).total;
}

extern "C" int cgnn_spmm(const cgnn_csr *A, int dtype, const void *X, void *Y, int64_t F,
                         int accumulate, int kernel, void *workspace, size_t workspace_bytes,
                         cgnn_stream_t stream) {
    int rc = check_csr(A, "cgnn_spmm");
    if (rc != CGNN_OK) return rc;
    CGNN_REQUIRE(F >= 0, "cgnn_spmm: F must be non-negative");
    if (A->rows == 0 || F == 0) return CGNN_OK;
    CGNN_REQUIRE(Y != nullptr, "cgnn_spmm: Y is null");
    CGNN_REQUIRE(A->nnz == 0 || X != nullptr, "cgnn_spmm: X is null");
    CGNN_REQUIRE(kernel >= CGNN_SPMM_AUTO && kernel <= CGNN_SPMM_NNZ, "cgnn_spmm: unknown kernel id");
    if (dtype == CGNN_F32)
        return spmm_typed<float>(A, X, nullptr, 0, nullptr, Y, F, accumulate, kernel, MODE_VAL, workspace,
                                 workspace_bytes, stream);
    if (dtype == CGNN_F64)
        return spmm_typed<double>(A, X, nullptr, 0, nullptr, Y, F, accumulate, kernel, MODE_VAL, workspace,
                                  workspace_bytes, stream);
    return fail(CGNN_EUNSUPPORTED, "cgnn_spmm: dtype must be f32 or f64");
}

extern "C" int cgnn_spmm_dual(const cgnn_csr *A, int64_t split, int dtype, const void *X0, const void *X1,
                              void *Y, int64_t F, int kernel, void *workspace, size_t workspace_bytes,
                              cgnn_stream_t stream) {
    int rc = check_csr(A, "cgnn_spmm_dual");
    if (rc != CGNN_OK) return rc;
    CGNN_REQUIRE(F >= 0, "cgnn_spmm_dual: F must be non-negative");
    CGNN_REQUIRE(split >= 0 && split <= A->cols, "cgnn_spmm_dual: split must be in [0, cols]");
    if (A->rows == 0 || F == 0) return CGNN_OK;
    CGNN_REQUIRE(Y != nullptr, "cgnn_spmm_dual: Y is null");
    CGNN_REQUIRE(A->nnz == 0 || ((split == 0 || X0 != nullptr) && (split == A->cols || X1 != nullptr)),
                 "cgnn_spmm_dual: a source matrix is null");
    CGNN_REQUIRE(kernel >= CGNN_SPMM_AUTO && kernel <= CGNN_SPMM_NNZ, "cgnn_spmm_dual: unknown kernel id");
    if (dtype == CGNN_F32)
        return spmm_typed<float>(A, X0, X1, split, nullptr, Y, F, 0, kernel, MODE_DUAL, workspace, workspace_bytes,
                                 stream);
    if (dtype == CGNN_F64)
        return spmm_typed<double>(A, X0, X1, split, nullptr, Y, F, 0, kernel, MODE_DUAL, workspace, workspace_bytes,
                                  stream);
    return fail(CGNN_EUNSUPPORTED, "cgnn_spmm_dual: dtype must be f32 or f64");
}

extern "C" int cgnn_csr_prepare_i64(int64_t rows, int64_t nnz, const int64_t *rowptr64,
                                    const int64_t *col64, int32_t *rowptr32, int32_t *col32,
                                    int32_t *rowidx, cgnn_stream_t stream) {
    const int64_t lim = (int64_t)INT32_MAX - 65536;
    CGNN_REQUIRE(rows >= 0 && nnz >= 0 && rows < lim && nnz < lim, "cgnn_csr_prepare_i64: sizes must be in [0, 2^31 - 65536)");
    CGNN_REQUIRE(rowptr64 != nullptr, "cgnn_csr_prepare_i64: rowptr is null");
    if (rowptr32) {
        hipLaunchKernelGGL(narrow_i64_kernel, dim3(grid_for(rows + 1)), dim3(kBlock), 0, stream, rowptr64,
                           rowptr32, rows + 1);
    }
    if (col32 && nnz > 0) {
        CGNN_REQUIRE(col64 != nullptr, "cgnn_csr_prepare_i64: col is null");
        hipLaunchKernelGGL(narrow_i64_kernel, dim3(grid_for(nnz)), dim3(kBlock), 0, stream, col64, col32, nnz);
    }
    if (rowidx && nnz > 0) {
        hipLaunchKernelGGL(expand_rows_kernel<int64_t>, dim3(grid_for(nnz)), dim3(kBlock), 0, stream,
                           rowptr64, rows, nnz, rowidx);
    }
    return check_launch("csr_prepare");
}

extern "C" int cgnn_narrow_ids(int64_t n, const int64_t *ids, int64_t groups, int32_t *narrow, int32_t *bad_id,
                               cgnn_stream_t stream) {
    const int64_t lim = (int64_t)INT32_MAX - 65536;
    CGNN_REQUIRE(n >= 0 && n < lim && groups >= 1 && groups < lim, "cgnn_narrow_ids: sizes must be in [0, 2^31 - 65536), at least one group");
    if (n == 0) return CGNN_OK;
    CGNN_REQUIRE(ids && narrow, "cgnn_narrow_ids: null array");
    hipLaunchKernelGGL(narrow_ids_kernel, dim3(grid_for(n)), dim3(kBlock), 0, stream, ids, n, groups, narrow, bad_id);
    return check_launch("narrow_ids");
}

extern "C" int cgnn_csr_compose_columns(int64_t nnz, const int32_t *colidx, int64_t first_cols, const int32_t *narrow_ids,
                                        int32_t *out, cgnn_stream_t stream) {
    const int64_t lim = (int64_t)INT32_MAX - 65536;
    CGNN_REQUIRE(nnz >= 0 && nnz < lim && first_cols >= 0 && first_cols < lim, "cgnn_csr_compose_columns: sizes must be in [0, 2^31 - 65536)");
    if (nnz == 0) return CGNN_OK;
    CGNN_REQUIRE(colidx && narrow_ids && out, "cgnn_csr_compose_columns: null array");
    CGNN_REQUIRE((reinterpret_cast<uintptr_t>(colidx) | reinterpret_cast<uintptr_t>(out)) % 16 == 0,
                 "cgnn_csr_compose_columns: colidx and out must be 16-byte aligned");
    hipLaunchKernelGGL(compose_columns_kernel, dim3(grid_for((nnz + 3) / 4)), dim3(kBlock), 0, stream, colidx, nnz, first_cols,
                       narrow_ids, out);
    return check_launch("csr_compose_columns");
}

extern "C" int cgnn_spmm_run_starts(const cgnn_csr *A, int32_t *run_start, cgnn_stream_t stream) {
    int rc = check_csr(A, "cgnn_spmm_run_starts");
    if (rc != CGNN_OK) return rc;
    CGNN_REQUIRE(run_start != nullptr, "cgnn_spmm_run_starts: null array");
    CGNN_REQUIRE(A->nnz == 0 || A->rowidx != nullptr, "cgnn_spmm_run_starts: the block needs rowidx");
    const int seg = seg_len(A);
    const int64_t n = ceil_div(A->nnz, seg) + 1;
    hipLaunchKernelGGL(run_starts_kernel, dim3((unsigned)ceil_div(n, kBlock)), dim3(kBlock), 0, stream, A->rowptr,
                       A->rowidx, (int32_t)A->nnz, seg, n, run_start);
    return check_launch("spmm_run_starts");
}

extern "C" int cgnn_csr_expand_rows(int64_t rows, int64_t nnz, const int32_t *rowptr, int32_t *rowidx,
                                    cgnn_stream_t stream) {
    const int64_t lim = (int64_t)INT32_MAX - 65536;
    CGNN_REQUIRE(rows >= 0 && nnz >= 0 && rows < lim && nnz < lim, "cgnn_csr_expand_rows: sizes must be in [0, 2^31 - 65536)");
    if (nnz == 0) return CGNN_OK;
    CGNN_REQUIRE(rowptr && rowidx, "cgnn_csr_expand_rows: null array");
    hipLaunchKernelGGL(expand_rows_kernel<int32_t>, dim3(grid_for(nnz)), dim3(kBlock), 0, stream, rowptr,
                       rows, nnz, rowidx);
    return check_launch("csr_expand_rows");
}
