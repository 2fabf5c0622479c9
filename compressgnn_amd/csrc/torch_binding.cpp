// `compressgnn_runtime`: the Python-visible operator module, with the operator names,
// argument order and error behaviour of the reference's extension
// (ZhengChenCS/CompressGNN src/runtime/csrc/function.cpp:9-21).  Host code only: every
// computation is a call into libcgnn_hip.so through the C ABI
// (include/compressgnn_abi.h); torch supplies tensors, the caching allocator and the
// current stream.  There is no CPU implementation behind these operators: CPU tensors
// are rejected with an error.
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <hip/hip_runtime_api.h>
#include <torch/extension.h>

#include <deque>
#include <memory>
#include <mutex>
#include <sstream>
#include <map>
#include <string>
#include <tuple>
#include <vector>

#include "compressgnn_abi.h"

namespace {

using torch::Tensor;

void ok(int rc, const char *what) {
    TORCH_CHECK(rc == CGNN_OK, what, ": ", cgnn_last_error());
}

cgnn_stream_t current_stream(const Tensor &t) {
    return reinterpret_cast<cgnn_stream_t>(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream());
}

int dtype_code(const Tensor &t) {
    TORCH_CHECK(t.scalar_type() == torch::kFloat32 || t.scalar_type() == torch::kFloat64,
                "Only float32 and float64 are supported");
    return t.scalar_type() == torch::kFloat32 ? CGNN_F32 : CGNN_F64;
}

void require_gpu(const Tensor &t, const char *name) {
    TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor: this build of compressgnn_runtime has no CPU operators");
}

// ----------------------------------------------------------------- CSR blocks ----

// Scratch memory of the nnz schedule (the carry rows), grown to the largest request and kept.
// A block owns one by default; the blocks of a propagation plan share one, since their
// products follow each other on one stream.  Two streams that run products over the same
// scratch at the same time would overwrite each other's carries: a caller who does that
// gives each stream a plan (or a block) of its own.
struct Scratch {
    Tensor buf;
    Tensor get(size_t bytes, const Tensor &like) {
        if (!buf.defined() || (size_t)buf.numel() < bytes || buf.device() != like.device())
            buf = torch::empty({(int64_t)std::max<size_t>(bytes, 1)}, like.options().dtype(torch::kUInt8));
        return buf;
    }
};

// A CSR block resident on the device in the layout the kernels read (int32 indices,
// row of every non-zero).  Built once per graph block.
struct DeviceCsr {
    int64_t rows = 0, cols = 0, nnz = 0;
    Tensor rowptr, colidx, rowidx, val;
    Tensor rowmap;  // optional: stored row g is output row rowmap[g]
    int64_t out_rows = 0;  // rows of the output: `rows`, or more when only the rows with entries are stored (rule levels)
    int32_t max_row_nnz = 0;
    int32_t seg_nnz = 0;
    Tensor cut_rows, empty_rows;  // the rows the runs of the nnz schedule cut / the rows without entries
    Tensor run_start;  // nnz schedule: where every run begins (made with rowidx)
    std::shared_ptr<Scratch> scratch = std::make_shared<Scratch>();

    cgnn_csr view() const {
        cgnn_csr a{};
        a.rows = rows;
        a.cols = cols;
        a.nnz = nnz;
        a.rowptr = rowptr.data_ptr<int32_t>();
        a.colidx = nnz ? colidx.data_ptr<int32_t>() : nullptr;
        a.rowidx = (nnz && rowidx.defined()) ? rowidx.data_ptr<int32_t>() : nullptr;
        a.val = (nnz && val.defined()) ? val.data_ptr() : nullptr;
        a.max_row_nnz = max_row_nnz;
        a.seg_nnz = seg_nnz;
        a.rowmap = rowmap.defined() ? rowmap.data_ptr<int32_t>() : nullptr;
        a.run_start = run_start.defined() ? run_start.data_ptr<int32_t>() : nullptr;
        if (cut_rows.defined()) {
            a.cut_rows = cut_rows.data_ptr<int32_t>();  // a tensor without entries gives a pointer that is never read
            a.n_cut_rows = (int32_t)cut_rows.numel();
            a.empty_rows = empty_rows.data_ptr<int32_t>();
            a.n_empty_rows = (int32_t)empty_rows.numel();
        }
        return a;
    }

    // Which rows the runs cut depends on rowptr and the run length only: found once, here (two
    // small host reads at build time), so that the fix-up pass of every product goes straight to them.
    void list_rows() {
        cut_rows = Tensor();
        empty_rows = Tensor();
        if (rows == 0 || nnz == 0) return;
        cgnn_csr a = view();
        const int64_t K = cgnn_spmm_run_length(&a);
        Tensor start = rowptr.slice(0, 0, rows).to(torch::kInt64), end = rowptr.slice(0, 1, rows + 1).to(torch::kInt64);
        // a row of at most K entries is never cut; a longer one is cut at the multiples of K inside it
        Tensor cut = ((end - start) > K).logical_and((torch::floor_divide(start, K) + 1) * K < end);
        Tensor found = torch::nonzero(cut).flatten().to(torch::kInt32);
        Tensor none = torch::nonzero(start == end).flatten().to(torch::kInt32);
        // a pointer is needed even for an empty list (NULL means "no lists"): keep one entry of storage
        auto pad = [](const Tensor &t) { return t.numel() ? t : torch::zeros({1}, t.options()).narrow(0, 0, 0); };
        cut_rows = pad(found.contiguous());
        empty_rows = pad(none.contiguous());
    }

    // rowidx (the row of every non-zero, as large as colidx) is read by the nnz schedule only:
    // it is made when a product first resolves to that schedule, on the product's stream.
    // So is the table of run starts, which belongs to a run length as the row lists do.
    void ensure_rowidx(int kernel) {
        if (nnz == 0 || (rowidx.defined() && run_start.defined())) return;
        if (cgnn_spmm_schedule(rows, nnz, max_row_nnz, kernel) != CGNN_SPMM_NNZ) return;
        auto stream = reinterpret_cast<cgnn_stream_t>(
            c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(rowptr.device().index()).stream());
        if (!rowidx.defined()) {
            rowidx = torch::empty({nnz}, rowptr.options());
            ok(cgnn_csr_expand_rows(rows, nnz, rowptr.data_ptr<int32_t>(), rowidx.data_ptr<int32_t>(), stream),
               "csr_expand_rows");
        }
        cgnn_csr a = view();
        const int64_t K = cgnn_spmm_run_length(&a);
        Tensor starts = torch::empty({(nnz + K - 1) / K + 1}, rowptr.options());
        ok(cgnn_spmm_run_starts(&a, starts.data_ptr<int32_t>(), stream), "spmm_run_starts");
        run_start = starts;
    }

    Tensor workspace(int64_t F, int dtype, int kernel, size_t *bytes) {
        ensure_rowidx(kernel);
        cgnn_csr a = view();
        *bytes = cgnn_spmm_workspace_bytes(&a, F, dtype, kernel);
        return scratch->get(*bytes, rowptr);
    }
};

// rowptr/col: int64 or int32 tensors on any device; value: float tensor or undefined.
std::shared_ptr<DeviceCsr> make_csr(Tensor rowptr, Tensor col, c10::optional<Tensor> value, int64_t rows,
                                    int64_t cols, torch::Device device, int64_t seg_nnz,
                                    c10::optional<Tensor> rowmap = c10::nullopt, bool with_row_lists = true,
                                    int64_t out_rows = -1) {
    TORCH_CHECK(device.is_cuda(), "DeviceCsr lives on a GPU");
    TORCH_CHECK(rowptr.dim() == 1 && col.dim() == 1 && rowptr.numel() == rows + 1, "rowptr must have rows+1 entries");
    auto blk = std::make_shared<DeviceCsr>();
    blk->rows = rows;
    blk->out_rows = out_rows < 0 ? rows : out_rows;
    TORCH_CHECK(blk->out_rows >= rows && (blk->out_rows == rows || (rowmap.has_value() && rowmap->defined())),
                "a block that stores fewer rows than its output has needs a rowmap");
    blk->cols = cols;
    blk->nnz = col.numel();
    blk->seg_nnz = (int32_t)seg_nnz;
    const int64_t lim = (int64_t)INT32_MAX - 65536;
    TORCH_CHECK(rows < lim && cols < lim && blk->nnz < lim, "block exceeds the int32 index range of the kernels");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(device);
    Tensor rp = rowptr.to(device).contiguous();
    Tensor ci = col.to(device).contiguous();
    auto i32 = torch::TensorOptions().device(device).dtype(torch::kInt32);
    if (rp.scalar_type() == torch::kInt64) {
        blk->rowptr = torch::empty({rows + 1}, i32);
        blk->colidx = torch::empty({blk->nnz}, i32);
        TORCH_CHECK(ci.scalar_type() == torch::kInt64, "rowptr and col must have the same integer type");
        ok(cgnn_csr_prepare_i64(rows, blk->nnz, rp.data_ptr<int64_t>(), blk->nnz ? ci.data_ptr<int64_t>() : nullptr,
                                blk->rowptr.data_ptr<int32_t>(), blk->nnz ? blk->colidx.data_ptr<int32_t>() : nullptr,
                                nullptr, current_stream(rp)),
           "csr_prepare");
    } else {
        TORCH_CHECK(rp.scalar_type() == torch::kInt32 && ci.scalar_type() == torch::kInt32,
                    "rowptr/col must be int64 or int32");
        blk->rowptr = rp;
        blk->colidx = ci;
    }
    if (value.has_value() && value->defined()) {
        TORCH_CHECK(value->numel() == blk->nnz, "value must have one entry per non-zero");
        blk->val = value->to(device).contiguous();
    }
    if (rowmap.has_value() && rowmap->defined()) {
        TORCH_CHECK(rowmap->dim() == 1 && rowmap->numel() == rows, "rowmap must have one entry per row");
        blk->rowmap = rowmap->to(device).to(torch::kInt32).contiguous();
    }
    if (rows > 0) {
        Tensor lens = blk->rowptr.slice(0, 1, rows + 1) - blk->rowptr.slice(0, 0, rows);
        blk->max_row_nnz = lens.max().item<int32_t>();  // one host read per block, at build time
    }
    if (with_row_lists) blk->list_rows();
    return blk;
}

int kernel_of_method(const std::string &method) {
    // The reference's GPU method strings (src/runtime/csrc/sparse/cuda/spmm_gpu.cu:27-31) and
    // its two CPU ones are accepted.  Its layers pick among them from (nnz, width) alone
    // (layer/CompressgnnSPMM.py:14-19) and, for instance, ask for "rowbalance_rowcache" on every
    // large block, power-law in-lists included, where a lane group per row is many times slower
    // here.  They are therefore hints: the schedule is chosen from the block's row lengths, as
    // for "auto".  "row_schedule" and "nnz_schedule" are this build's names for a forced
    // schedule (bit-exact comparisons with a sequential sum, measurements).
    static const char *const hints[] = {"auto", "rowbalance", "rowbalance_parreduce", "rowbalance_seqreduce",
                                        "rowbalance_rowcache", "nnzbalance", "nnzbalance_parreduce",
                                        "nnzbalance_seqreduce", "nnzbalance_rowcache"};
    for (const char *h : hints)
        if (method == h) return CGNN_SPMM_AUTO;
    if (method == "row_schedule") return CGNN_SPMM_ROW;
    if (method == "nnz_schedule") return CGNN_SPMM_NNZ;
    TORCH_CHECK(false, "Invalid SpMM method: ", method);
}

// out (+)= A * mat.  `out` undefined: a fresh [rows, F] tensor is returned.
Tensor block_spmm(DeviceCsr &A, const Tensor &mat, c10::optional<Tensor> optional_out, int kernel) {
    require_gpu(mat, "mat");
    TORCH_CHECK(mat.is_contiguous(), "mat must be contiguous");
    TORCH_CHECK(mat.dim() == 2, "mat must be a matrix");
    TORCH_CHECK(mat.size(0) == A.cols, "mat has ", mat.size(0), " rows, the block has ", A.cols, " columns");
    TORCH_CHECK(!A.val.defined() || A.val.scalar_type() == mat.scalar_type(), "value and mat must have the same dtype");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(mat.device());
    const int64_t F = mat.size(1);
    const int dtype = dtype_code(mat);
    Tensor out;
    int accumulate = 0;
    if (optional_out.has_value() && optional_out->defined()) {
        // like the reference (spmm_gpu.cu:20-22) a non-contiguous out is copied, so the
        // caller must use the returned tensor
        out = optional_out->contiguous();
        require_gpu(out, "out");
        TORCH_CHECK(out.dim() == 2 && out.size(0) == A.out_rows && out.size(1) == F && out.scalar_type() == mat.scalar_type(),
                    "out must be [rows, F] of mat's dtype");
        accumulate = 1;
    } else if (A.out_rows != A.rows) {
        out = torch::zeros({A.out_rows, F}, mat.options());  // the rows that are not stored have no entries
    } else {
        out = torch::empty({A.rows, F}, mat.options());
    }
    if (A.rows == 0 || F == 0) return out;
    size_t bytes = 0;
    Tensor ws = A.workspace(F, dtype, kernel, &bytes);
    cgnn_csr a = A.view();
    ok(cgnn_spmm(&a, dtype, mat.data_ptr(), out.data_ptr(), F, accumulate, kernel, ws.data_ptr(), bytes,
                 current_stream(mat)),
       "spmm");
    return out;
}

// spmm_func of the reference (src/runtime/csrc/sparse/spmm.cpp:11-22): CSR given as
// int64 tensors, prepared on every call.  Graph blocks that are used repeatedly should
// be wrapped in a DeviceCsr once instead.
Tensor spmm_func(Tensor vlist, Tensor elist, Tensor value, Tensor mat, std::string method,
                 c10::optional<Tensor> optional_out) {
    require_gpu(mat, "mat");
    require_gpu(vlist, "vlist");
    require_gpu(elist, "elist");
    require_gpu(value, "value");
    const int kernel = kernel_of_method(method);
    TORCH_CHECK(vlist.scalar_type() == torch::kInt64 && elist.scalar_type() == torch::kInt64,
                "vlist and elist must be int64");
    auto blk = make_csr(vlist, elist, value, vlist.size(-1) - 1, mat.size(0), mat.device(), 0, c10::nullopt, false);
    return block_spmm(*blk, mat, optional_out, kernel);
}

// ------------------------------------------------------- compressed propagation ----

// Optional per-stage timing with HIP events on the stream the kernels run on.  Events
// are recorded only around the stages named in `timed` ("*" = all), so a timed region
// can carry one pair of events per step without disturbing the rest.
struct StageTimer {
    struct Rec {
        std::string name;
        hipEvent_t begin, end;
    };
    std::vector<std::string> timed;
    std::vector<Rec> recs;
    // An event pair costs the stream a few microseconds of idle time on either side of the stage, so
    // a caller that times a loop may ask for every n-th pass of a stage only.
    int64_t every = 1;
    std::map<std::string, int64_t> passes;

    bool wants(const std::string &name) const {
        for (auto &t : timed)
            if (t == "*" || t == name) return true;
        return false;
    }
    int open(const std::string &name, hipStream_t stream) {
        if (!wants(name)) return -1;
        if (passes[name]++ % std::max<int64_t>(every, 1) != 0) return -1;
        Rec r{name, nullptr, nullptr};
        TORCH_CHECK(hipEventCreate(&r.begin) == hipSuccess && hipEventCreate(&r.end) == hipSuccess, "hipEventCreate failed");
        TORCH_CHECK(hipEventRecord(r.begin, stream) == hipSuccess, "hipEventRecord failed");
        recs.push_back(r);
        return (int)recs.size() - 1;
    }
    void close(int id, hipStream_t stream) {
        if (id >= 0) TORCH_CHECK(hipEventRecord(recs[id].end, stream) == hipSuccess, "hipEventRecord failed");
    }
    // (stage, milliseconds) of every recorded interval; call after the stream is idle.
    std::vector<std::pair<std::string, double>> take() {
        std::vector<std::pair<std::string, double>> out;
        for (auto &r : recs) {
            float ms = 0;
            TORCH_CHECK(hipEventSynchronize(r.end) == hipSuccess, "hipEventSynchronize failed");
            TORCH_CHECK(hipEventElapsedTime(&ms, r.begin, r.end) == hipSuccess, "hipEventElapsedTime failed");
            out.emplace_back(r.name, (double)ms);
            hipEventDestroy(r.begin);
            hipEventDestroy(r.end);
        }
        recs.clear();
        return out;
    }
    ~StageTimer() {
        for (auto &r : recs) {
            hipEventDestroy(r.begin);
            hipEventDestroy(r.end);
        }
    }
};

// The device form of a CompressGraph (loader/compress_graph.py:6-43 of the reference):
// the three vertex/rule blocks, the rule levels and their transposes.
struct PropagationPlan {
    // rule stage and rule levels, forward and backward
    std::shared_ptr<DeviceCsr> r2v, v2r_t;
    std::vector<std::shared_ptr<DeviceCsr>> r2r, r2r_t;
    // [v2v | v2r] and [v2v^T | r2v^T]: the vertex stage of forward / backward in one pass
    std::shared_ptr<DeviceCsr> vertex_stage, vertex_stage_t;
    // the four blocks of the vertex stages on their own: only for the two-launch form
    // (fuse_final = false); a plan without them holds the graph once
    std::shared_ptr<DeviceCsr> v2v, v2r, v2v_t, r2v_t;
    int64_t V = 0, R = 0;
    bool fuse_final = true;  // last two stages in one pass (cgnn_spmm_dual)
    int kernel = CGNN_SPMM_AUTO;
    std::shared_ptr<Scratch> scratch = std::make_shared<Scratch>();
    StageTimer timer;
    // The forward blocks with their vertex columns sent through a cluster assignment
    // (propagate_forward_gathered), kept for the index tensors they were made for: an
    // assignment lasts until the next refresh, and a model may hold one per layer.
    struct Composed {
        c10::weak_intrusive_ptr<c10::TensorImpl> index;
        uint32_t version;
        int64_t groups;
        std::shared_ptr<DeviceCsr> rules, stage;
    };
    std::deque<Composed> composed;

    void adopt(const std::shared_ptr<DeviceCsr> &block) {
        if (block) block->scratch = scratch;
    }
    bool fused() const { return fuse_final && vertex_stage && vertex_stage_t; }
    void require_split_blocks() const {
        TORCH_CHECK(v2v && v2r && v2v_t && r2v_t,
                    "this plan holds the fused vertex stages only; the two-launch form needs the v2v, v2r, v2v_t and "
                    "r2v_t blocks (graph.keep_split_blocks = True before graph.plan())");
    }
};

Tensor timed_spmm(PropagationPlan &p, const std::string &stage, DeviceCsr &A, const Tensor &mat,
                  c10::optional<Tensor> out) {
    hipStream_t stream = reinterpret_cast<hipStream_t>(current_stream(mat));
    const int id = p.timer.open(stage, stream);
    Tensor r = block_spmm(A, mat, out, p.kernel);
    p.timer.close(id, stream);
    return r;
}

Tensor final_stage(PropagationPlan &p, const std::string &prefix, DeviceCsr *merged,
                   const std::shared_ptr<DeviceCsr> &from_rules, const Tensor &rule_x,
                   const std::shared_ptr<DeviceCsr> &from_vertices, const Tensor &x) {
    const int64_t F = x.size(1);
    if (p.fuse_final && merged != nullptr) {
        Tensor out = torch::empty({merged->rows, F}, x.options());
        if (out.numel() == 0) return out;
        const int dtype = dtype_code(x);
        size_t bytes = 0;
        Tensor ws = merged->workspace(F, dtype, p.kernel, &bytes);
        hipStream_t stream = reinterpret_cast<hipStream_t>(current_stream(x));
        const int id = p.timer.open(prefix + "final", stream);
        cgnn_csr a = merged->view();
        ok(cgnn_spmm_dual(&a, p.V, dtype, x.data_ptr(), rule_x.data_ptr(), out.data_ptr(), F, p.kernel,
                          ws.data_ptr(), bytes, current_stream(x)),
           "spmm_dual");
        p.timer.close(id, stream);
        return out;
    }
    p.require_split_blocks();
    Tensor out = timed_spmm(p, prefix + "from_rules", *from_rules, rule_x, c10::nullopt);
    return timed_spmm(p, prefix + "from_vertices", *from_vertices, x, out);
}

// layer/CompressgnnSPMM.py:43-62 of the reference.  Stage names: fwd.rules (r2v),
// fwd.level<i>, fwd.final (v2r + v2v fused) or fwd.from_rules / fwd.from_vertices.
Tensor propagate_forward(PropagationPlan &p, Tensor x) {
    require_gpu(x, "x");
    TORCH_CHECK(x.dim() == 2 && x.size(0) == p.V, "x must be [vertex_cnt, F]");
    x = x.contiguous();
    c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
    Tensor rule_out = timed_spmm(p, "fwd.rules", *p.r2v, x, c10::nullopt);
    for (size_t i = 0; i < p.r2r.size(); ++i)
        rule_out = timed_spmm(p, "fwd.level" + std::to_string(i), *p.r2r[i], rule_out, rule_out);
    return final_stage(p, "fwd.", p.vertex_stage.get(), p.v2r, rule_out, p.v2v, x);
}

// A copy of a block that shares everything but the column numbers: the columns below
// `first_cols` go through `index` (cgnn_csr_compose_columns).
std::shared_ptr<DeviceCsr> compose_block(const DeviceCsr &A, const Tensor &narrow, int64_t first_cols, int64_t cols) {
    auto blk = std::make_shared<DeviceCsr>(A);
    blk->cols = cols;
    if (A.nnz > 0) {
        blk->colidx = torch::empty_like(A.colidx);
        ok(cgnn_csr_compose_columns(A.nnz, A.colidx.data_ptr<int32_t>(), first_cols, narrow.data_ptr<int32_t>(),
                                    blk->colidx.data_ptr<int32_t>(), current_stream(narrow)),
           "csr_compose_columns");
    }
    return blk;
}

// out = A * reps[index] over the compressed graph without reps[index]: the forward chain of
// propagate_forward on blocks whose vertex columns name the representative of the vertex.
// reps: [groups, F]; index: int64 [vertex_cnt] with values in [0, groups).  The same sums in the
// same order as propagate_forward(reps.index_select(0, index)): the same bits.  The composed
// blocks are made on the first call for an index tensor (one host read: the ids are checked)
// and kept until that tensor is written to or freed.  Stage names: fwd.rules, fwd.level<i>, fwd.final.
Tensor propagate_forward_gathered(PropagationPlan &p, Tensor reps, Tensor index) {
    require_gpu(reps, "reps");
    require_gpu(index, "index");
    TORCH_CHECK(reps.dim() == 2 && reps.size(0) >= 1, "reps must be [groups, F] with at least one group");
    TORCH_CHECK(index.dim() == 1 && index.numel() == p.V && index.scalar_type() == torch::kInt64 && index.is_contiguous() &&
                    index.device() == reps.device(),
                "index must be a contiguous int64 tensor [vertex_cnt] on the device of reps");
    TORCH_CHECK(p.fused(), "propagation from representatives needs the fused vertex stage (plan.fuse_final = True)");
    reps = reps.contiguous();
    c10::hip::HIPGuardMasqueradingAsCUDA guard(reps.device());
    const int64_t groups = reps.size(0), F = reps.size(1);
    std::shared_ptr<DeviceCsr> rules, stage;
    for (auto it = p.composed.begin(); it != p.composed.end();) {
        if (it->index.expired()) {
            it = p.composed.erase(it);
            continue;
        }
        if (it->index._unsafe_get_target() == index.unsafeGetTensorImpl() && it->version == index._version() &&
            it->groups == groups) {
            rules = it->rules;
            stage = it->stage;
            break;
        }
        ++it;
    }
    if (!stage) {
        Tensor bad = torch::zeros({1}, index.options().dtype(torch::kInt32));
        Tensor narrow = torch::empty({p.V}, index.options().dtype(torch::kInt32));
        ok(cgnn_narrow_ids(p.V, index.data_ptr<int64_t>(), groups, narrow.data_ptr<int32_t>(), bad.data_ptr<int32_t>(),
                           current_stream(index)),
           "narrow_ids");
        rules = compose_block(*p.r2v, narrow, p.V, groups);
        stage = compose_block(*p.vertex_stage, narrow, p.V, p.vertex_stage->cols);
        TORCH_CHECK(bad.item<int32_t>() == 0, "propagation from representatives: the index holds a cluster id outside [0, ", groups, ")");
        if (!index.is_inference()) {
            p.composed.push_front(PropagationPlan::Composed{c10::weak_intrusive_ptr<c10::TensorImpl>(index.getIntrusivePtr()),
                                                           index._version(), groups, rules, stage});
            while (p.composed.size() > 4) p.composed.pop_back();
        }
    }
    Tensor rule_out = timed_spmm(p, "fwd.rules", *rules, reps, c10::nullopt);
    for (size_t i = 0; i < p.r2r.size(); ++i)
        rule_out = timed_spmm(p, "fwd.level" + std::to_string(i), *p.r2r[i], rule_out, rule_out);
    Tensor out = torch::empty({p.V, F}, reps.options());
    if (out.numel() == 0) return out;
    const int dtype = dtype_code(reps);
    size_t bytes = 0;
    Tensor ws = stage->workspace(F, dtype, p.kernel, &bytes);
    hipStream_t stream = reinterpret_cast<hipStream_t>(current_stream(reps));
    const int id = p.timer.open("fwd.final", stream);
    cgnn_csr a = stage->view();
    ok(cgnn_spmm_dual(&a, p.V, dtype, reps.data_ptr(), rule_out.data_ptr(), out.data_ptr(), F, p.kernel, ws.data_ptr(), bytes,
                      current_stream(reps)),
       "spmm_dual");
    p.timer.close(id, stream);
    return out;
}

// layer/CompressgnnSPMM.py:65-86 (the working branch, lines 80-85).  Stage names as in
// forward with the prefix bwd.
Tensor propagate_backward(PropagationPlan &p, Tensor grad) {
    require_gpu(grad, "grad");
    TORCH_CHECK(grad.dim() == 2 && grad.size(0) == p.V, "grad must be [vertex_cnt, F]");
    grad = grad.contiguous();
    c10::hip::HIPGuardMasqueradingAsCUDA guard(grad.device());
    Tensor rule_g = timed_spmm(p, "bwd.rules", *p.v2r_t, grad, c10::nullopt);
    for (size_t i = p.r2r_t.size(); i-- > 0;)
        rule_g = timed_spmm(p, "bwd.level" + std::to_string(i), *p.r2r_t[i], rule_g, rule_g);
    return final_stage(p, "bwd.", p.vertex_stage_t.get(), p.r2v_t, rule_g, p.v2v_t, grad);
}

// ---------------------------------------------------- transformation compression ----

// Operand checks of the transformation-compression operators.  Every operator names its
// operands once, as a row of Operand records, and `expect` reports the first one that does not
// fit, saying what was asked for and what arrived.
enum class Role { Features, Ids, Counts, Bias };

struct Operand {
    Role role;
    const char *name;
    const Tensor *tensor;
};

std::string seen(const Tensor &t) {
    std::ostringstream os;
    os << t.scalar_type() << t.sizes() << " on " << t.device() << (t.is_contiguous() ? "" : ", not contiguous");
    return os.str();
}

// `anchor`: the operand whose device (and, for floating operands, precision) the others share.
void expect(const char *op, const Tensor &anchor, std::initializer_list<Operand> operands) {
    for (const Operand &o : operands) {
        const Tensor &t = *o.tensor;
        bool fits = t.defined() && t.is_cuda() && t.is_contiguous() && t.device() == anchor.device();
        const char *asked = "";
        switch (o.role) {
            case Role::Features:
                asked = "a contiguous [rows, width] float32 or float64 matrix on the GPU";
                fits = fits && t.dim() == 2 && (t.scalar_type() == torch::kFloat32 || t.scalar_type() == torch::kFloat64) &&
                       t.scalar_type() == anchor.scalar_type();
                break;
            case Role::Ids:
                asked = "a contiguous int64 vector of cluster ids beside the features";
                fits = fits && t.dim() == 1 && t.scalar_type() == torch::kInt64;
                break;
            case Role::Counts:
                asked = "a contiguous int32 vector with at least the empty cluster 0, beside the features";
                fits = fits && t.dim() == 1 && t.scalar_type() == torch::kInt32 && t.numel() > 0;
                break;
            case Role::Bias:
                asked = "a contiguous vector of the features' precision, beside the features";
                fits = fits && t.dim() == 1 && t.scalar_type() == anchor.scalar_type();
                break;
        }
        TORCH_CHECK(fits, op, ": ", o.name, " has to be ", asked, "; it is ", t.defined() ? seen(t) : "undefined");
    }
}

// Number of hash buckets for `bits` sign bits.
int64_t buckets_for(const char *op, int64_t bits) {
    TORCH_CHECK(0 <= bits && bits <= 30, op, ": between 0 and 30 hyperplanes are supported, ", bits, " asked for");
    return int64_t(1) << bits;
}

// The hyperplanes of an assignment: one column per sign bit, one row per input feature.
void expect_planes(const char *op, const Tensor &input, const Tensor &planes, int64_t bits) {
    expect(op, input, {{Role::Features, "input", &input}, {Role::Features, "hyperplanes", &planes}});
    TORCH_CHECK(planes.size(0) == input.size(1) && planes.size(1) == bits, op, ": ", bits, " hyperplanes over ",
                input.size(1), " features make a [", input.size(1), ", ", bits, "] matrix, not ", planes.sizes());
    TORCH_CHECK(input.size(0) < INT_MAX, op, ": ", input.size(0), " rows do not fit the int32 cluster sizes");
}

// cluster_workspace_cuda (src/runtime/csrc/cluster/cuda/cluster_kernel.cu:111-117):
// [bucket counts int32[2^bits], prefix int32[2^bits], scan scratch uint8[...]].
std::vector<Tensor> cluster_workspace(Tensor input, int64_t bits) {
    const char *op = "cluster_workspace";
    expect(op, input, {{Role::Features, "input", &input}});
    const int64_t buckets = buckets_for(op, bits);
    c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
    auto ints = input.options().dtype(torch::kInt32);
    return {torch::empty({buckets}, ints), torch::empty({buckets}, ints),
            torch::empty({(int64_t)cgnn_lsh_scan_workspace_bytes((int)bits)}, input.options().dtype(torch::kUInt8))};
}

// Assignment and member lists of one refresh: ids [N] int64 (1-based), counts
// [active+1] int32 (entry 0 = 0), active, and the member lists (offsets [active+2], perm
// [N], sorted_id [N], and a host scalar with the size of the largest group).  The codes are grouped by a stable sort instead of bucket counters,
// so the result is the same as cluster_assign_cuda's (cluster_kernel.cu:118-153) whatever
// the distribution of the codes, and the member lists come with it.  The number of groups
// is at most min(N, 2^bits): every kernel runs on buffers of that bound, so the device
// never waits for the host; the one scalar read of a refresh (cluster_kernel.cu:146-147)
// comes last and only trims the views.
std::tuple<Tensor, Tensor, int64_t, std::vector<Tensor>> cluster_assign_members(Tensor input, Tensor planes,
                                                                                int64_t bits) {
    const char *op = "cluster_assign";
    const int64_t buckets = buckets_for(op, bits);
    expect_planes(op, input, planes, bits);
    c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
    const int64_t N = input.size(0);
    auto ints = input.options().dtype(torch::kInt32);
    Tensor ids = torch::empty({N}, input.options().dtype(torch::kInt64));
    Tensor perm = torch::empty({N}, ints), sorted_id = torch::empty({N}, ints);
    auto host_scalar = [](int64_t v) { return torch::full({1}, v, torch::TensorOptions().dtype(torch::kInt64)); };
    if (N == 0)
        return {ids, torch::zeros({1}, ints), 0, {torch::zeros({2}, ints), perm, sorted_id, host_scalar(0)}};
    const int64_t cap = std::min<int64_t>(N, buckets);
    Tensor raw = torch::empty({N}, ints);
    Tensor offsets = torch::empty({cap + 2}, ints), counts = torch::empty({cap + 1}, ints);
    Tensor summary_dev = torch::empty({2}, ints);  // number of groups, largest group
    auto stream = current_stream(input);
    ok(cgnn_lsh_hash(N, input.size(1), (int)bits, dtype_code(input), input.data_ptr(), planes.data_ptr(),
                     raw.data_ptr<int32_t>(), nullptr, stream),
       "lsh_hash");
    const size_t bytes = cgnn_lsh_group_workspace_bytes(N, (int)bits);
    Tensor ws = torch::empty({(int64_t)std::max<size_t>(bytes, 1)}, input.options().dtype(torch::kUInt8));
    ok(cgnn_lsh_group(N, (int)bits, raw.data_ptr<int32_t>(), ids.data_ptr<int64_t>(), offsets.data_ptr<int32_t>(),
                      perm.data_ptr<int32_t>(), sorted_id.data_ptr<int32_t>(), counts.data_ptr<int32_t>(),
                      summary_dev.data_ptr<int32_t>(), ws.data_ptr(), bytes, stream),
       "lsh_group");
    Tensor summary = summary_dev.cpu();  // the one host read of a refresh
    const int active = summary.data_ptr<int32_t>()[0];
    return {ids, counts.narrow(0, 0, active + 1), (int64_t)active,
            {offsets.narrow(0, 0, active + 2), perm, sorted_id, host_scalar(summary.data_ptr<int32_t>()[1])}};
}

// Member lists by the index tensor they belong to.  The operators with the reference's
// signatures (cluster_mean(input, index, count), cluster_reconstruct(reps, index, bias, relu), ...)
// receive an index and nothing else; the lists that go with it, and the knowledge that its ids
// were checked, are kept here so that only the first call on an index builds them (one host
// read), as the reference reads the host once per assignment (cluster_kernel.cu:147).  An entry
// names its tensor by a weak reference and the tensor's version counter: it is dropped when the
// tensor is freed and ignored once the tensor was written to.
struct MemberCache {
    struct Entry {
        c10::weak_intrusive_ptr<c10::TensorImpl> index;
        uint32_t version;
        int64_t groups;
        std::vector<Tensor> members;
    };
    static constexpr size_t kKeep = 8;
    std::deque<Entry> entries;
    std::mutex lock;

    bool find(const Tensor &index, int64_t groups, std::vector<Tensor> *out) {
        std::lock_guard<std::mutex> hold(lock);
        for (auto it = entries.begin(); it != entries.end();) {
            if (it->index.expired()) {
                it = entries.erase(it);
                continue;
            }
            if (it->index._unsafe_get_target() == index.unsafeGetTensorImpl() && it->version == index._version() &&
                (groups < 0 || it->groups == groups)) {
                *out = it->members;
                return true;
            }
            ++it;
        }
        return false;
    }
    void put(const Tensor &index, int64_t groups, std::vector<Tensor> members) {
        if (index.is_inference()) return;  // no version counter to tell a later write by
        std::lock_guard<std::mutex> hold(lock);
        entries.push_front(Entry{c10::weak_intrusive_ptr<c10::TensorImpl>(index.getIntrusivePtr()), index._version(),
                                 groups, std::move(members)});
        while (entries.size() > kKeep) entries.pop_back();
    }
};

MemberCache &member_cache() {
    static MemberCache cache;
    return cache;
}

// cluster_assign_cuda (cluster_kernel.cu:118-153).  The three tensors of cluster_workspace
// are accepted, and must be what cluster_workspace returns for these arguments; the grouping
// itself sorts the codes and no longer touches bucket counters.
std::tuple<Tensor, Tensor, int64_t> cluster_assign(Tensor input, Tensor planes, int64_t bits,
                                                   std::vector<Tensor> workspace) {
    const char *op = "cluster_assign";
    const int64_t buckets = buckets_for(op, bits);
    expect_planes(op, input, planes, bits);
    TORCH_CHECK(workspace.size() == 3, op, ": the workspace is the three tensors of cluster_workspace, ", workspace.size(),
                " given");
    const int64_t need[3] = {buckets, buckets, (int64_t)cgnn_lsh_scan_workspace_bytes((int)bits)};
    const torch::ScalarType kind[3] = {torch::kInt32, torch::kInt32, torch::kUInt8};
    for (int i = 0; i < 3; ++i) {
        const Tensor &w = workspace[i];
        const bool fits = w.defined() && w.device() == input.device() && w.dim() == 1 && w.is_contiguous() &&
                          w.scalar_type() == kind[i] && (i < 2 ? w.numel() == need[i] : w.numel() >= need[i]);
        TORCH_CHECK(fits, op, ": workspace[", i, "] has to be ", kind[i], "[", need[i], "] beside the input; it is ",
                    w.defined() ? seen(w) : "undefined");
    }
    auto grouped = cluster_assign_members(input, planes, bits);
    // the lists made along the way stay with the ids: the operators that are handed these ids
    // (and nothing else) find them again
    member_cache().put(std::get<0>(grouped), std::get<2>(grouped) + 1, std::get<3>(grouped));
    return {std::get<0>(grouped), std::get<1>(grouped), std::get<2>(grouped)};
}

// cluster_forward (src/runtime/csrc/cluster/cluster.cpp:12-30): int32 ids and the
// number of active buckets.
std::tuple<Tensor, int64_t> cluster_forward(Tensor input, Tensor random_vectors, int64_t param_h) {
    require_gpu(input, "input");
    auto grouped = cluster_assign_members(input, random_vectors, param_h);
    return {std::get<0>(grouped).to(torch::kInt32), std::get<2>(grouped)};
}

// One int32 on the device that the kernels set when they meet a cluster id that names no
// cluster; `raise` reads it (the only host read of these operators, made only for index
// tensors that do not come with member lists of this library's own making).
struct IdFlag {
    Tensor flag;
    explicit IdFlag(const Tensor &like) : flag(torch::zeros({1}, like.options().dtype(torch::kInt32))) {}
    int32_t *ptr() { return flag.data_ptr<int32_t>(); }
    void raise(const char *op, int64_t groups) {
        TORCH_CHECK(flag.item<int32_t>() == 0, op, ": the index holds a cluster id outside [0, ", groups, ")");
    }
};

// Member lists of `groups` clusters: [offsets int32[groups+1], perm int32[N], sorted_id int32[N]].
std::vector<Tensor> cluster_members(Tensor index, int64_t groups) {
    const char *op = "cluster_members";
    require_gpu(index, "index");
    expect(op, index, {{Role::Ids, "index", &index}});
    TORCH_CHECK(groups >= 1, op, ": at least the empty cluster 0 is needed, groups = ", groups);
    c10::hip::HIPGuardMasqueradingAsCUDA guard(index.device());
    const int64_t N = index.numel();
    auto i32 = index.options().dtype(torch::kInt32);
    Tensor offsets = torch::empty({groups + 1}, i32), perm = torch::empty({N}, i32), sorted = torch::empty({N}, i32);
    const size_t bytes = cgnn_cluster_members_workspace_bytes(N, groups);
    Tensor ws = torch::empty({(int64_t)std::max<size_t>(bytes, 1)}, index.options().dtype(torch::kUInt8));
    IdFlag bad(index);
    ok(cgnn_cluster_members(N, groups, N ? index.data_ptr<int64_t>() : nullptr, offsets.data_ptr<int32_t>(),
                            N ? perm.data_ptr<int32_t>() : nullptr, N ? sorted.data_ptr<int32_t>() : nullptr, bad.ptr(),
                            ws.data_ptr(), bytes, current_stream(index)),
       op);
    bad.raise(op, groups);
    return {offsets, perm, sorted};
}

// Member lists handed in by the caller ([offsets, perm, sorted_id] and optionally a host int64
// scalar with the size of the largest group), checked against the index they belong to.
bool has_members(const c10::optional<std::vector<Tensor>> &members) { return members.has_value() && !members->empty(); }

void expect_members(const char *op, const std::vector<Tensor> &m, const Tensor &index, int64_t groups) {
    TORCH_CHECK(m.size() == 3 || m.size() == 4, op, ": member lists are [offsets, perm, sorted_id] (+ largest group), ",
                m.size(), " tensors given");
    const int64_t want[3] = {groups + 1, index.numel(), index.numel()};
    const char *names[3] = {"offsets", "perm", "sorted_id"};
    for (int i = 0; i < 3; ++i)
        TORCH_CHECK(m[i].defined() && m[i].scalar_type() == torch::kInt32 && m[i].device() == index.device() &&
                        m[i].is_contiguous() && (groups < 0 && i == 0 ? true : m[i].numel() == want[i]),
                    op, ": member list '", names[i], "' has to be int32[", want[i], "] beside the index; it is ",
                    m[i].defined() ? seen(m[i]) : "undefined");
    if (m.size() == 4)
        TORCH_CHECK(!m[3].is_cuda() && m[3].numel() == 1 && m[3].scalar_type() == torch::kInt64, op,
                    ": the fourth member tensor is a host int64 scalar (size of the largest group)");
}

std::vector<Tensor> members_or_build(const char *op, const c10::optional<std::vector<Tensor>> &members,
                                     const Tensor &index, int64_t groups) {
    if (has_members(members)) {
        expect_members(op, *members, index, groups);
        return *members;
    }
    std::vector<Tensor> known;
    if (member_cache().find(index, groups, &known)) return known;
    known = cluster_members(index, groups);  // checks the ids: the one host read for this index
    member_cache().put(index, groups, known);
    return known;
}

int64_t largest_group(const std::vector<Tensor> &m) { return m.size() == 4 ? m[3].item<int64_t>() : 0; }

// cluster_mean_cuda (cluster_kernel.cu:158-170).  `members` (from cluster_members, for
// the same index) avoids rebuilding the member lists on every call.
Tensor cluster_mean(Tensor input, Tensor index, Tensor count, c10::optional<std::vector<Tensor>> members) {
    const char *op = "cluster_mean";
    expect(op, input, {{Role::Features, "input", &input}, {Role::Ids, "index", &index}, {Role::Counts, "count", &count}});
    TORCH_CHECK(index.numel() == input.size(0), op, ": ", input.size(0), " rows but ", index.numel(), " cluster ids");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
    const int64_t N = input.size(0), F = input.size(1), groups = count.numel();
    if (input.numel() == 0) return torch::zeros({groups, F}, input.options());
    auto m = members_or_build(op, members, index, groups);
    Tensor out = torch::empty({groups, F}, input.options());
    const size_t bytes = cgnn_cluster_mean_workspace_bytes(N, F, groups, dtype_code(input));
    Tensor ws = torch::empty({(int64_t)std::max<size_t>(bytes, 1)}, input.options().dtype(torch::kUInt8));
    ok(cgnn_cluster_mean(N, F, groups, largest_group(m), dtype_code(input), input.data_ptr(), m[0].data_ptr<int32_t>(),
                         m[1].data_ptr<int32_t>(), m[2].data_ptr<int32_t>(), count.data_ptr<int32_t>(), out.data_ptr(),
                         ws.data_ptr(), bytes, current_stream(input)),
       op);
    return out;
}

// The order in which a gather produces its rows: the member list `perm` when the caller has one
// or an earlier operator on the same index has left one (`held` keeps it alive for the call).
// An index met for the first time, without lists, is an index from outside the assignment
// operators: its ids are checked by the gather itself (one host read) and its lists are built
// for the calls that follow.
const int32_t *production_order(const char *op, const c10::optional<std::vector<Tensor>> &members, const Tensor &index,
                                int64_t groups, std::vector<Tensor> *held) {
    if (has_members(members)) {
        expect_members(op, *members, index, -1);
        return (*members)[1].data_ptr<int32_t>();
    }
    if (member_cache().find(index, groups, held)) return (*held)[1].data_ptr<int32_t>();
    return nullptr;
}

// After a gather over an index that had no lists: the flag is read (the ids are then known to be
// good) and the lists are made, so that later operators on this index read nothing.
void remember_checked_index(const char *op, IdFlag &bad, const Tensor &index, int64_t groups) {
    bad.raise(op, groups);
    if (groups >= 1) member_cache().put(index, groups, cluster_members(index, groups));
}

// cluster_mean_backward_cuda (cluster_kernel.cu:171-181).
Tensor cluster_mean_backward(Tensor grad, Tensor index, Tensor count, c10::optional<std::vector<Tensor>> members) {
    const char *op = "cluster_mean_backward";
    expect(op, grad, {{Role::Features, "grad", &grad}, {Role::Ids, "index", &index}, {Role::Counts, "count", &count}});
    TORCH_CHECK(grad.size(0) == count.numel(), op, ": ", grad.size(0), " gradient rows for ", count.numel(), " clusters");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(grad.device());
    Tensor out = torch::empty({index.numel(), grad.size(1)}, grad.options());
    if (out.numel() == 0) return out;
    std::vector<Tensor> held;
    const int32_t *perm = production_order(op, members, index, count.numel(), &held);
    c10::optional<IdFlag> bad;
    if (perm == nullptr) bad.emplace(index);
    ok(cgnn_cluster_mean_backward(index.numel(), grad.size(1), count.numel(), dtype_code(grad), grad.data_ptr(),
                                  index.data_ptr<int64_t>(), count.data_ptr<int32_t>(), perm, out.data_ptr(),
                                  bad ? bad->ptr() : nullptr, current_stream(grad)),
       op);
    if (bad) remember_checked_index(op, *bad, index, count.numel());
    return out;
}

// cluster_reconstruct_cuda (cluster_kernel.cu:182-195).
Tensor cluster_reconstruct(Tensor reps, Tensor index, c10::optional<Tensor> bias, bool relu,
                           c10::optional<std::vector<Tensor>> members) {
    const char *op = "cluster_reconstruct";
    expect(op, reps, {{Role::Features, "representatives", &reps}, {Role::Ids, "index", &index}});
    if (bias.has_value()) {
        expect(op, reps, {{Role::Bias, "bias", &*bias}});
        TORCH_CHECK(bias->numel() == reps.size(1), op, ": a bias of ", bias->numel(), " entries for rows of ", reps.size(1));
    }
    TORCH_CHECK(index.numel() == 0 || reps.size(0) > 0, op, ": rows to reconstruct but no representatives");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(reps.device());
    Tensor out = torch::empty({index.numel(), reps.size(1)}, reps.options());
    if (out.numel() == 0) return out;
    std::vector<Tensor> held;
    const int32_t *perm = production_order(op, members, index, reps.size(0), &held);
    c10::optional<IdFlag> bad;
    if (perm == nullptr) bad.emplace(index);
    ok(cgnn_reconstruct(index.numel(), reps.size(1), reps.size(0), dtype_code(reps), reps.data_ptr(),
                        index.data_ptr<int64_t>(), perm, bias.has_value() ? bias->data_ptr() : nullptr, relu ? 1 : 0,
                        out.data_ptr(), bad ? bad->ptr() : nullptr, current_stream(reps)),
       op);
    if (bad) remember_checked_index(op, *bad, index, reps.size(0));
    return out;
}

// cluster_reconstruct_backward_cuda (cluster_kernel.cu:196-208).
Tensor cluster_reconstruct_backward(Tensor grad, Tensor index, Tensor output, int64_t groups, bool relu,
                                    c10::optional<std::vector<Tensor>> members) {
    const char *op = "cluster_reconstruct_backward";
    expect(op, grad, {{Role::Features, "grad", &grad}, {Role::Ids, "index", &index}, {Role::Features, "output", &output}});
    TORCH_CHECK(groups >= 0, op, ": groups = ", groups);
    TORCH_CHECK(output.sizes() == grad.sizes(), op, ": the saved output is ", output.sizes(), ", the gradient ", grad.sizes());
    TORCH_CHECK(index.numel() == grad.size(0), op, ": ", grad.size(0), " rows but ", index.numel(), " cluster ids");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(grad.device());
    const int64_t N = grad.size(0), F = grad.size(1);
    if (grad.numel() == 0 || groups == 0) return torch::zeros({groups, F}, grad.options());
    auto m = members_or_build(op, members, index, groups);
    Tensor out = torch::empty({groups, F}, grad.options());
    const size_t bytes = cgnn_cluster_mean_workspace_bytes(N, F, groups, dtype_code(grad));
    Tensor ws = torch::empty({(int64_t)std::max<size_t>(bytes, 1)}, grad.options().dtype(torch::kUInt8));
    ok(cgnn_reconstruct_backward(N, F, groups, largest_group(m), dtype_code(grad), grad.data_ptr(), output.data_ptr(),
                                 m[0].data_ptr<int32_t>(), m[1].data_ptr<int32_t>(), m[2].data_ptr<int32_t>(),
                                 relu ? 1 : 0, out.data_ptr(), ws.data_ptr(), bytes, current_stream(grad)),
       op);
    return out;
}

// The ReLU form of cluster_reconstruct that also returns the sign of every output element as one
// bit: (rows [N, F], signs int32 [N, ceil(F / 32)]).  A layer keeps the signs for its backward pass
// instead of the rows (the reference keeps the rows: layer/CompressgnnReconstruct.py:16-22).
std::tuple<Tensor, Tensor> cluster_reconstruct_signs(Tensor reps, Tensor index, c10::optional<Tensor> bias,
                                                     c10::optional<std::vector<Tensor>> members) {
    const char *op = "cluster_reconstruct_signs";
    expect(op, reps, {{Role::Features, "representatives", &reps}, {Role::Ids, "index", &index}});
    if (bias.has_value()) {
        expect(op, reps, {{Role::Bias, "bias", &*bias}});
        TORCH_CHECK(bias->numel() == reps.size(1), op, ": a bias of ", bias->numel(), " entries for rows of ", reps.size(1));
    }
    TORCH_CHECK(index.numel() == 0 || reps.size(0) > 0, op, ": rows to reconstruct but no representatives");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(reps.device());
    const int64_t N = index.numel(), F = reps.size(1);
    Tensor out = torch::empty({N, F}, reps.options());
    Tensor signs = torch::empty({N, cgnn_sign_words(F)}, reps.options().dtype(torch::kInt32));
    if (out.numel() == 0) return {out, signs};
    std::vector<Tensor> held;
    const int32_t *perm = production_order(op, members, index, reps.size(0), &held);
    c10::optional<IdFlag> bad;
    if (perm == nullptr) bad.emplace(index);
    ok(cgnn_reconstruct_signs(N, F, reps.size(0), dtype_code(reps), reps.data_ptr(), index.data_ptr<int64_t>(), perm,
                              bias.has_value() ? bias->data_ptr() : nullptr, out.data_ptr(),
                              reinterpret_cast<uint32_t *>(signs.data_ptr<int32_t>()), bad ? bad->ptr() : nullptr,
                              current_stream(reps)),
       op);
    if (bad) remember_checked_index(op, *bad, index, reps.size(0));
    return {out, signs};
}

// cluster_reconstruct_backward with relu = true, the mask taken from the signs above.
Tensor cluster_reconstruct_backward_signs(Tensor grad, Tensor index, Tensor signs, int64_t groups,
                                          c10::optional<std::vector<Tensor>> members) {
    const char *op = "cluster_reconstruct_backward_signs";
    expect(op, grad, {{Role::Features, "grad", &grad}, {Role::Ids, "index", &index}});
    TORCH_CHECK(groups >= 0, op, ": groups = ", groups);
    TORCH_CHECK(index.numel() == grad.size(0), op, ": ", grad.size(0), " rows but ", index.numel(), " cluster ids");
    const int64_t N = grad.size(0), F = grad.size(1);
    TORCH_CHECK(signs.device() == grad.device() && signs.scalar_type() == torch::kInt32 && signs.is_contiguous() &&
                    signs.dim() == 2 && signs.size(0) == N && signs.size(1) == cgnn_sign_words(F),
                op, ": signs must be a contiguous int32 tensor [", N, ", ", cgnn_sign_words(F), "] on the device of grad");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(grad.device());
    if (grad.numel() == 0 || groups == 0) return torch::zeros({groups, F}, grad.options());
    auto m = members_or_build(op, members, index, groups);
    Tensor out = torch::empty({groups, F}, grad.options());
    const size_t bytes = cgnn_cluster_mean_workspace_bytes(N, F, groups, dtype_code(grad));
    Tensor ws = torch::empty({(int64_t)std::max<size_t>(bytes, 1)}, grad.options().dtype(torch::kUInt8));
    ok(cgnn_reconstruct_backward_signs(N, F, groups, largest_group(m), dtype_code(grad), grad.data_ptr(),
                                       reinterpret_cast<const uint32_t *>(signs.data_ptr<int32_t>()),
                                       m[0].data_ptr<int32_t>(), m[1].data_ptr<int32_t>(), m[2].data_ptr<int32_t>(),
                                       out.data_ptr(), ws.data_ptr(), bytes, current_stream(grad)),
       op);
    return out;
}

// (colptr, row, value) of a block held as int64 tensors on a GPU: the CSR of its transpose,
// in the order SparseTensor.csc() gives.  The one host read (a flag for columns out of
// range) comes after the last kernel.
std::tuple<Tensor, Tensor, c10::optional<Tensor>> csr_transpose(Tensor rowptr, Tensor col, c10::optional<Tensor> value,
                                                                int64_t cols) {
    TORCH_CHECK(rowptr.is_cuda() && col.is_cuda(), "csr_transpose: tensors must be on a GPU");
    TORCH_CHECK(rowptr.scalar_type() == torch::kInt64 && col.scalar_type() == torch::kInt64,
                "csr_transpose: rowptr and col must be int64");
    TORCH_CHECK(rowptr.dim() == 1 && col.dim() == 1 && rowptr.numel() >= 1 && cols >= 0, "csr_transpose: bad shapes");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(rowptr.device());
    const int64_t rows = rowptr.numel() - 1, nnz = col.numel();
    Tensor rp = rowptr.contiguous(), ci = col.contiguous();
    Tensor val;
    int dtype = CGNN_F32;
    if (value.has_value() && value->defined()) {
        TORCH_CHECK(value->is_cuda() && value->dim() == 1 && value->numel() == nnz,
                    "csr_transpose: value must have one entry per non-zero");
        TORCH_CHECK(value->scalar_type() == torch::kFloat32 || value->scalar_type() == torch::kFloat64,
                    "csr_transpose: value must be float32 or float64");
        val = value->contiguous();
        dtype = dtype_code(val);
    }
    Tensor colptr = torch::empty({cols + 1}, rp.options());
    Tensor row = torch::empty({nnz}, rp.options());
    Tensor tval = val.defined() ? torch::empty_like(val) : Tensor();
    Tensor bad = torch::empty({1}, rp.options().dtype(torch::kInt32));
    const size_t bytes = cgnn_csr_transpose_workspace_bytes(nnz);
    Tensor ws = torch::empty({(int64_t)std::max<size_t>(bytes, 1)}, rp.options().dtype(torch::kUInt8));
    ok(cgnn_csr_transpose_device(rows, cols, nnz, rp.data_ptr<int64_t>(), nnz ? ci.data_ptr<int64_t>() : nullptr, dtype,
                                 val.defined() && nnz ? val.data_ptr() : nullptr, colptr.data_ptr<int64_t>(),
                                 nnz ? row.data_ptr<int64_t>() : nullptr, tval.defined() && nnz ? tval.data_ptr() : nullptr,
                                 bad.data_ptr<int32_t>(), ws.data_ptr(), bytes, current_stream(rp)),
       "csr_transpose");
    TORCH_CHECK(bad.item<int32_t>() == 0, "csr_transpose: column out of range [0, ", cols, ")");
    if (tval.defined()) return {colptr, row, tval};
    return {colptr, row, c10::nullopt};
}

// ------------------------------------------------ neighbour sampling (compressed graph) ----

// The host side of a sampling call: sizes the outputs of every layer (two scalar reads per
// layer: neighbours of the layer, vertices it adds) and strings the device entry points
// together.  neighbor_sample_sim_impl / neighbor_sample_ori_impl of the reference's module
// compressgnn_sample (src/sample/csrc/neighbor_sample.h:27-131, 134-211), on GPU tensors.
struct SampleGraph {
    cgnn_sample_graph view{};
    std::vector<Tensor> keep;  // contiguous int64 tensors behind the pointers
    torch::Device device = torch::kCPU;

    const int64_t *hold(const Tensor &t, const char *name) {
        TORCH_CHECK(t.defined() && t.is_cuda() && t.scalar_type() == torch::kInt64 && t.dim() == 1,
                    "neighbor_sample: ", name, " has to be a one-dimensional int64 GPU tensor");
        TORCH_CHECK(keep.empty() || t.device() == device, "neighbor_sample: ", name, " lives on another device");
        device = t.device();
        keep.push_back(t.contiguous());
        return keep.back().numel() ? keep.back().data_ptr<int64_t>() : nullptr;
    }
};

std::tuple<Tensor, Tensor, Tensor> run_sampler(SampleGraph &G, const Tensor &input_node,
                                               const std::vector<int64_t> &num_neighbors, int64_t seed, bool swap_roles) {
    const char *op = "neighbor_sample";
    const cgnn_sample_graph &g = G.view;
    TORCH_CHECK(input_node.is_cuda() && input_node.device() == G.device && input_node.scalar_type() == torch::kInt64 &&
                    input_node.dim() == 1,
                op, ": input_node has to be a one-dimensional int64 tensor beside the graph");
    for (int64_t fan : num_neighbors) TORCH_CHECK(fan >= 0, op, ": a fan-out of ", fan);
    c10::hip::HIPGuardMasqueradingAsCUDA guard(G.device);
    auto stream = current_stream(input_node);
    auto i64 = input_node.options();
    auto i32 = input_node.options().dtype(torch::kInt32);
    auto u8 = input_node.options().dtype(torch::kUInt8);
    const Tensor input = input_node.contiguous();
    const int64_t n_input = input.numel();
    Tensor local_of = torch::empty({std::max<int64_t>(g.vertex_cnt, 1)}, i32), seen_at = torch::empty_like(local_of);
    Tensor status = torch::empty({1}, i32);
    ok(cgnn_sample_relabel_begin(g.vertex_cnt, n_input, n_input ? input.data_ptr<int64_t>() : nullptr,
                                 local_of.data_ptr<int32_t>(), seen_at.data_ptr<int32_t>(), status.data_ptr<int32_t>(),
                                 stream),
       op);
    auto raise_on = [&](int32_t code) {
        TORCH_CHECK_INDEX(code != CGNN_SAMPLE_OUT_OF_RANGE, "Neighbor index out of range");
        TORCH_CHECK(code != CGNN_SAMPLE_BAD_VERTEX, op, ": a vertex id outside [0, ", g.vertex_cnt, ")");
        TORCH_CHECK(code != CGNN_SAMPLE_TOO_MANY, op, ": a layer of more than 2^31 - 2 neighbours");
    };
    Tensor samples = input.clone();
    std::vector<Tensor> sources, numbers;
    int64_t begin = 0, end = n_input;
    for (size_t layer = 0; layer < num_neighbors.size(); ++layer) {
        const int64_t n = end - begin, fanout = num_neighbors[layer];
        if (n == 0) break;
        Tensor frontier = samples.narrow(0, begin, n);
        Tensor counts = torch::empty({n}, i32), offsets = torch::empty({n + 1}, i32);
        ok(cgnn_sample_count(&g, n, frontier.data_ptr<int64_t>(), fanout, counts.data_ptr<int32_t>(),
                             status.data_ptr<int32_t>(), stream),
           op);
        const size_t sum_bytes = cgnn_exclusive_sum_workspace_bytes(n);
        Tensor sum_ws = torch::empty({(int64_t)std::max<size_t>(sum_bytes, 1)}, u8);
        ok(cgnn_exclusive_sum_i32(n, counts.data_ptr<int32_t>(), offsets.data_ptr<int32_t>(), status.data_ptr<int32_t>(),
                                  sum_ws.data_ptr(), sum_bytes, stream),
           op);
        // first scalar read of the layer: its size (and whether anything went wrong so far)
        Tensor head = torch::stack({offsets[n], status[0]}).cpu();
        raise_on(head.data_ptr<int32_t>()[1]);
        const int64_t total = head.data_ptr<int32_t>()[0];
        Tensor neighbors = torch::empty({total}, i64), source = torch::empty({total}, i64), picks = torch::empty({total}, i64);
        Tensor number = torch::empty({total}, i64), added = torch::empty({1}, i64);
        Tensor grown = torch::empty({end + total}, i64);
        grown.narrow(0, 0, end).copy_(samples);
        if (total > 0) {
            ok(cgnn_sample_fill(&g, n, frontier.data_ptr<int64_t>(), fanout, offsets.data_ptr<int32_t>(), begin,
                                (int64_t)layer, (uint64_t)seed, neighbors.data_ptr<int64_t>(), source.data_ptr<int64_t>(),
                                picks.data_ptr<int64_t>(), status.data_ptr<int32_t>(), stream),
               op);
        }
        const size_t bytes = cgnn_sample_relabel_workspace_bytes(total);
        Tensor ws = torch::empty({(int64_t)std::max<size_t>(bytes, 1)}, u8);
        ok(cgnn_sample_relabel(total, total ? neighbors.data_ptr<int64_t>() : nullptr, end, local_of.data_ptr<int32_t>(),
                               seen_at.data_ptr<int32_t>(), grown.data_ptr<int64_t>(), total ? number.data_ptr<int64_t>() : nullptr,
                               added.data_ptr<int64_t>(), ws.data_ptr(), bytes, stream),
           op);
        // second scalar read: how many vertices the layer added
        Tensor tail = torch::stack({added[0], status[0].to(torch::kInt64)}).cpu();
        raise_on((int32_t)tail.data_ptr<int64_t>()[1]);
        const int64_t fresh = tail.data_ptr<int64_t>()[0];
        samples = grown.narrow(0, 0, end + fresh);
        sources.push_back(source);
        numbers.push_back(number);
        begin = end;
        end += fresh;
    }
    Tensor empty = torch::empty({0}, i64);
    Tensor of_source = sources.empty() ? empty : torch::cat(sources), of_neighbor = numbers.empty() ? empty : torch::cat(numbers);
    // (samples, rows, cols): the compressed form reports (source, neighbour), the plain form the reverse
    if (swap_roles) return {samples.clone(), of_neighbor, of_source};
    return {samples.clone(), of_source, of_neighbor};
}

std::tuple<Tensor, Tensor, Tensor> neighbor_sample_cg_sim(Tensor v2v_vlist, Tensor v2v_elist, Tensor v2r_vlist,
                                                          Tensor v2r_elist, Tensor r2v_vlist, Tensor r2v_elist,
                                                          std::vector<Tensor> r2r_vlist, std::vector<Tensor> r2r_elist,
                                                          Tensor v_degree, Tensor r_degree, Tensor input_node,
                                                          std::vector<int64_t> num_neighbors, int64_t seed) {
    SampleGraph G;
    cgnn_sample_graph &g = G.view;
    g.v2v_ptr = G.hold(v2v_vlist, "v2v_vlist");
    g.v2v_idx = G.hold(v2v_elist, "v2v_elist");
    g.v2r_ptr = G.hold(v2r_vlist, "v2r_vlist");
    g.v2r_idx = G.hold(v2r_elist, "v2r_elist");
    g.r2v_ptr = G.hold(r2v_vlist, "r2v_vlist");
    g.r2v_idx = G.hold(r2v_elist, "r2v_elist");
    TORCH_CHECK(r2r_vlist.size() == r2r_elist.size() && r2r_vlist.size() <= CGNN_SAMPLE_MAX_LEVELS,
                "neighbor_sample: ", r2r_vlist.size(), " row-pointer and ", r2r_elist.size(), " column tensors of rule levels (at most ",
                CGNN_SAMPLE_MAX_LEVELS, " levels)");
    g.levels = (int32_t)r2r_vlist.size();
    g.vertex_cnt = v2v_vlist.numel() - 1;
    g.rule_cnt = r2v_vlist.numel() - 1;
    TORCH_CHECK(g.vertex_cnt >= 0 && g.rule_cnt >= 0 && v2r_vlist.numel() == g.vertex_cnt + 1,
                "neighbor_sample: row pointers have to hold vertex_cnt + 1 (v2v, v2r) and rule_cnt + 1 (r2v) entries");
    for (int k = 0; k < g.levels; ++k) {
        TORCH_CHECK(r2r_vlist[k].numel() == g.rule_cnt + 1, "neighbor_sample: level ", k, " has to hold rule_cnt + 1 row pointers");
        g.r2r_ptr[k] = G.hold(r2r_vlist[k], "r2r_vlist");
        g.r2r_idx[k] = G.hold(r2r_elist[k], "r2r_elist");
    }
    TORCH_CHECK(v_degree.numel() == g.vertex_cnt && r_degree.numel() == g.rule_cnt,
                "neighbor_sample: one expanded degree per vertex and per rule");
    g.v_degree = G.hold(v_degree, "v_degree");
    g.r_degree = G.hold(r_degree, "r_degree");
    return run_sampler(G, input_node, num_neighbors, seed, false);
}

std::tuple<Tensor, Tensor, Tensor> neighbor_sample_ori_impl(Tensor colptr, Tensor row, Tensor input_node,
                                                            std::vector<int64_t> num_neighbors, int64_t seed) {
    SampleGraph G;
    cgnn_sample_graph &g = G.view;
    g.v2v_ptr = G.hold(colptr, "colptr");
    g.v2v_idx = G.hold(row, "row");
    g.vertex_cnt = colptr.numel() - 1;
    TORCH_CHECK(g.vertex_cnt >= 0, "neighbor_sample: colptr has to hold vertex_cnt + 1 entries");
    return run_sampler(G, input_node, num_neighbors, seed, true);
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    namespace py = pybind11;
    m.doc() = "CompressGNN runtime operators for MI355X (HIP kernels behind a C ABI)";
    // the reference's operator set (src/runtime/csrc/function.cpp:10-20)
    m.def("spmm_func", &spmm_func, "spmm function", py::arg("vlist"), py::arg("elist"), py::arg("value"),
          py::arg("mat"), py::arg("method"), py::arg("optional_out") = py::none());
    m.def("cluster_forward", &cluster_forward, "CompressGNN cluster forward");
    m.def("cluster_workspace", &cluster_workspace);
    m.def("cluster_assign", &cluster_assign);
    m.def("cluster_assign_members", &cluster_assign_members,
          "(ids, counts, active, [offsets, perm, sorted_id]) of one assignment refresh");
    m.def("cluster_mean", &cluster_mean, py::arg("input"), py::arg("index"), py::arg("count"),
          py::arg("members") = py::none());
    m.def("cluster_mean_backward", &cluster_mean_backward, py::arg("grad"), py::arg("index"), py::arg("count"),
          py::arg("members") = py::none());
    m.def("cluster_reconstruct", &cluster_reconstruct, py::arg("reps"), py::arg("index"), py::arg("bias"),
          py::arg("relu"), py::arg("members") = py::none());
    m.def("cluster_reconstruct_backward", &cluster_reconstruct_backward, py::arg("grad"), py::arg("index"),
          py::arg("output"), py::arg("groups"), py::arg("relu"), py::arg("members") = py::none());
    // the reference's sampler module (src/sample/csrc/function.cpp:7-9), here on GPU tensors; `seed` keys
    // the counter-based generator of the random positions
    m.def("neighbor_sample_cg_sim", &neighbor_sample_cg_sim, "Neighbor Sample with CompressGraph Format",
          py::arg("v2v_vlist"), py::arg("v2v_elist"), py::arg("v2r_vlist"), py::arg("v2r_elist"), py::arg("r2v_vlist"),
          py::arg("r2v_elist"), py::arg("r2r_vlist"), py::arg("r2r_elist"), py::arg("v_degree"), py::arg("r_degree"),
          py::arg("input_node"), py::arg("num_neighbors"), py::arg("seed") = 0);
    m.def("neighbor_sample_ori_impl", &neighbor_sample_ori_impl, "Neighbor Sample with Normal Graph Format",
          py::arg("colptr"), py::arg("row"), py::arg("input_node"), py::arg("num_neighbors"), py::arg("seed") = 0);
    // additions of this build
    m.def("cluster_members", &cluster_members, "member lists (offsets, perm, sorted_id) of the clusters");
    m.def("cluster_reconstruct_signs", &cluster_reconstruct_signs,
          "cluster_reconstruct with ReLU -> (rows, one sign bit per element)", py::arg("reps"), py::arg("index"),
          py::arg("bias"), py::arg("members") = py::none());
    m.def("cluster_reconstruct_backward_signs", &cluster_reconstruct_backward_signs,
          "cluster_reconstruct_backward with ReLU, masked by the sign bits", py::arg("grad"), py::arg("index"),
          py::arg("signs"), py::arg("groups"), py::arg("members") = py::none());
    m.def("csr_transpose", &csr_transpose, "CSR -> CSC of an int64 block on the GPU, SparseTensor.csc() order",
          py::arg("rowptr"), py::arg("col"), py::arg("value"), py::arg("cols"));
    m.def("version", []() { return std::string(cgnn_version()); });
    py::class_<DeviceCsr, std::shared_ptr<DeviceCsr>>(m, "DeviceCsr")
        .def(py::init([](Tensor rowptr, Tensor col, c10::optional<Tensor> value, int64_t rows, int64_t cols,
                         torch::Device device, int64_t seg_nnz, c10::optional<Tensor> rowmap, int64_t out_rows) {
                 return make_csr(rowptr, col, value, rows, cols, device, seg_nnz, rowmap, true, out_rows);
             }),
             py::arg("rowptr"), py::arg("col"), py::arg("value"), py::arg("rows"), py::arg("cols"),
             py::arg("device"), py::arg("seg_nnz") = 0, py::arg("rowmap") = py::none(), py::arg("out_rows") = -1)
        .def_readonly("rowmap", &DeviceCsr::rowmap)
        .def_readonly("out_rows", &DeviceCsr::out_rows)
        .def_readonly("rows", &DeviceCsr::rows)
        .def_readonly("cols", &DeviceCsr::cols)
        .def_readonly("nnz", &DeviceCsr::nnz)
        .def_readonly("max_row_nnz", &DeviceCsr::max_row_nnz)
        .def_property("seg_nnz", [](DeviceCsr &self) { return self.seg_nnz; },
                      [](DeviceCsr &self, int32_t seg) {
                          self.seg_nnz = seg;
                          self.run_start = Tensor();  // made again by the next product
                          if (self.cut_rows.defined()) self.list_rows();  // the lists belong to a run length
                      })
        .def_readonly("cut_rows", &DeviceCsr::cut_rows)
        .def_readonly("run_start", &DeviceCsr::run_start)
        .def_readonly("empty_rows", &DeviceCsr::empty_rows)
        .def_readonly("rowptr", &DeviceCsr::rowptr)
        .def_readonly("colidx", &DeviceCsr::colidx)
        .def_readonly("rowidx", &DeviceCsr::rowidx)
        .def_readonly("val", &DeviceCsr::val)
        .def("spmm",
             [](DeviceCsr &self, Tensor mat, c10::optional<Tensor> out, std::string method) {
                 return block_spmm(self, mat, out, kernel_of_method(method));
             },
             py::arg("mat"), py::arg("out") = py::none(), py::arg("method") = "auto");
    py::class_<PropagationPlan, std::shared_ptr<PropagationPlan>>(m, "PropagationPlan")
        .def(py::init([](int64_t V, int64_t R, std::shared_ptr<DeviceCsr> r2v, std::vector<std::shared_ptr<DeviceCsr>> r2r,
                         std::shared_ptr<DeviceCsr> v2r_t, std::vector<std::shared_ptr<DeviceCsr>> r2r_t) {
                 auto p = std::make_shared<PropagationPlan>();
                 TORCH_CHECK(r2v && v2r_t, "the rule stages r2v and v2r_t are required");
                 TORCH_CHECK(r2r.size() == r2r_t.size(), "levels and transposed levels differ in number");
                 TORCH_CHECK(r2v->rows == R && r2v->cols == V && v2r_t->rows == R && v2r_t->cols == V,
                             "the rule stages must be [rule_cnt, vertex_cnt]");
                 p->V = V; p->R = R;
                 p->r2v = r2v; p->r2r = r2r; p->v2r_t = v2r_t; p->r2r_t = r2r_t;
                 p->adopt(r2v); p->adopt(v2r_t);
                 for (auto &b : r2r) p->adopt(b);
                 for (auto &b : r2r_t) p->adopt(b);
                 return p;
             }),
             py::arg("vertex_cnt"), py::arg("rule_cnt"), py::arg("r2v"), py::arg("r2r"), py::arg("v2r_t"), py::arg("r2r_t"))
        .def("set_vertex_stages",
             [](PropagationPlan &p, std::shared_ptr<DeviceCsr> fwd, std::shared_ptr<DeviceCsr> bwd) {
                 TORCH_CHECK(fwd && bwd && fwd->rows == p.V && bwd->rows == p.V && fwd->cols == p.V + p.R &&
                                 bwd->cols == p.V + p.R,
                             "a vertex stage is [vertex_cnt, vertex_cnt + rule_cnt]");
                 p.vertex_stage = fwd; p.vertex_stage_t = bwd;
                 p.adopt(fwd); p.adopt(bwd);
             })
        .def("set_split_blocks",
             [](PropagationPlan &p, std::shared_ptr<DeviceCsr> v2v, std::shared_ptr<DeviceCsr> v2r,
                std::shared_ptr<DeviceCsr> v2v_t, std::shared_ptr<DeviceCsr> r2v_t) {
                 p.v2v = v2v; p.v2r = v2r; p.v2v_t = v2v_t; p.r2v_t = r2v_t;
                 p.adopt(v2v); p.adopt(v2r); p.adopt(v2v_t); p.adopt(r2v_t);
                 p.require_split_blocks();
             })
        .def_property("fuse_final", [](PropagationPlan &p) { return p.fuse_final; },
                      [](PropagationPlan &p, bool fuse) {
                          if (!fuse) p.require_split_blocks();
                          else TORCH_CHECK(p.vertex_stage && p.vertex_stage_t, "this plan has no fused vertex stages");
                          p.fuse_final = fuse;
                      })
        .def_readonly("vertex_stage", &PropagationPlan::vertex_stage)
        .def_readonly("vertex_stage_t", &PropagationPlan::vertex_stage_t)
        .def_property_readonly("scratch_bytes",
                               [](PropagationPlan &p) { return p.scratch->buf.defined() ? p.scratch->buf.numel() : 0; })
        .def_property("method",
                      [](PropagationPlan &p) { return p.kernel == CGNN_SPMM_ROW ? "row_schedule" : p.kernel == CGNN_SPMM_NNZ ? "nnz_schedule" : "auto"; },
                      [](PropagationPlan &p, std::string mth) { p.kernel = kernel_of_method(mth); })
        .def_property("timed_stages", [](PropagationPlan &p) { return p.timer.timed; },
                      [](PropagationPlan &p, std::vector<std::string> names) { p.timer.timed = names; })
        .def_property("timed_every", [](PropagationPlan &p) { return p.timer.every; },
                      [](PropagationPlan &p, int64_t n) {
                          TORCH_CHECK(n >= 1, "timed_every must be at least 1");
                          p.timer.every = n;
                          p.timer.passes.clear();
                      })
        .def("take_stage_times", [](PropagationPlan &p) { return p.timer.take(); })
        .def_readonly("v2v", &PropagationPlan::v2v)
        .def_readonly("v2r", &PropagationPlan::v2r)
        .def_readonly("r2v", &PropagationPlan::r2v)
        .def_readonly("r2r", &PropagationPlan::r2r)
        .def_readonly("v2v_t", &PropagationPlan::v2v_t)
        .def_readonly("v2r_t", &PropagationPlan::v2r_t)
        .def_readonly("r2v_t", &PropagationPlan::r2v_t)
        .def_readonly("r2r_t", &PropagationPlan::r2r_t)
        .def("forward", &propagate_forward)
        .def("forward_gathered", &propagate_forward_gathered, py::arg("reps"), py::arg("index"),
             "out = A * reps[index] without the [vertex_cnt, F] matrix reps[index]")
        .def("backward", &propagate_backward);
}
