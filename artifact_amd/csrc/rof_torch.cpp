// Compiled drop-in for the upstream `ROF` extension module (ROF/reuse_conv/reuse_conv.cpp:121-365): the same seven
// operators -- SAG, GNNA_forward / GNNA_backward, reuse_forward_v1 / reuse_backward_v1, reuse_forward_v2 /
// reuse_backward_v2 -- with upstream's positional signatures, CHECK_INPUT messages and return shapes, written
// against the C ABI of librof.so (include/rof.h) only.  PyTorch supplies device memory, the current stream and the
// dense update (torch::mm exactly where upstream calls it, reuse_conv_kernel.cu:302,382-383); the aggregation is
// rof_aggregate_epilogue.  The plan tensors are re-laid out on first use and cached by storage address, element
// count and version counter (upstream treats them as immutable and shares them across layers and passes,
// reuse_conv.py:40-43); `dimWorker` and `warpPerBlock` are hints of upstream's warp-per-part scheme and unused.
//
// Built by artifact_amd/build.py into artifact_amd/_ROF*.so; artifact_amd/ROF.py is the same interface in Python
// over ctypes, and tests/test_gpu_compiled_module.py holds the two bit for bit against each other.
#include <torch/extension.h>

#include <c10/hip/HIPStream.h>

#include <cstdlib>
#include <cstring>
#include <list>
#include <map>
#include <memory>
#include <tuple>
#include <vector>

#include "rof.h"
#include "rof_bench.h"

namespace {

#define CHECK_CUDA(x) TORCH_CHECK(x.device().is_cuda(), #x " must be a CUDA tensor")
#define CHECK_CONTIGUOUS(x) TORCH_CHECK(x.is_contiguous(), #x " must be contiguous")
#define CHECK_INPUT(x) \
    CHECK_CUDA(x);     \
    CHECK_CONTIGUOUS(x)

void rof_check(int rc, const char *what) {
    if (rc == ROF_OK) return;
    std::string msg = std::string("librof: ") + what + ": " + rof_strerror(rc);
    if (rc == ROF_ERR_DEVICE || rc == ROF_ERR_UNSUPPORTED) msg += std::string(" (") + rof_last_device_error() + ")";
    TORCH_CHECK(false, msg);
}

void *current_stream() { return (void *)c10::hip::getCurrentHIPStream().stream(); }

// lanes one gathered fp32 row occupies in the kernel (rof_layout_opts.lanes_per_row)
int lanes_per_row(int64_t feat) {
    static const int kChoices[] = {4, 8, 10, 12, 16, 20, 32, 64};
    const int64_t need = (feat + 3) / 4;
    for (int c : kChoices)
        if (c >= need) return c;
    return 64;
}

struct Layout {
    rof_layout *h = nullptr;
    torch::Tensor workspace;          // partial-sum rows, grown on demand
    const void *deg_ptr = nullptr;    // degree vector the weights were last set from
    int64_t deg_version = -1;
    torch::Tensor deg_keep;
    ~Layout() { rof_layout_free(h); }
};

// One plan in one of upstream's three tensor formats; a device layout per width class, built when first needed.
struct Plan {
    int kind = 0;   // 0: GNNA parts, 1: v1, 2: v2
    int part_size = 0;
    int64_t nodes = 0;
    std::vector<torch::Tensor> host;   // the plan tensors on the host (int32, contiguous)
    std::vector<torch::Tensor> keep;   // the device tensors whose addresses are the cache key
    std::map<int, std::unique_ptr<Layout>> by_lanes;   // by width class: 2 * lanes per row + (rows of >= 1024 bytes)

    Layout &get(int64_t feat) {
        const int lpr = lanes_per_row(feat);
        // one row per wavefront covers every width from 81 floats up: rows of 1024 bytes and more are a class of
        // their own (they are cut finer), like in the Python layer's LayoutFamily
        const int row_bytes = lpr == 64 ? (feat * 4 >= 1024 ? 1024 : 512) : 0;
        const int cls = lpr * 2 + (row_bytes == 1024);
        auto found = by_lanes.find(cls);
        if (found != by_lanes.end()) return *found->second;
        rof_layout_opts o;
        memset(&o, 0, sizeof(o));
        o.lanes_per_row = lpr;
        o.elem_bytes = 4;
        o.row_bytes = row_bytes;
        std::unique_ptr<Layout> lay(new Layout);
        lay->h = build(o);
        if (autotune_wanted()) autotune(lay, o, feat);
        return *(by_lanes[cls] = std::move(lay));
    }

    // the plan re-laid out with the given options
    rof_layout *build(rof_layout_opts o) {
        auto p = [this](size_t i) { return host[i].numel() ? host[i].data_ptr<int32_t>() : nullptr; };
        rof_layout *h = nullptr;
        int rc;
        if (kind == 0) {
            rc = rof_layout_from_parts(p(0), host[1].data_ptr<int32_t>(), p(2), host[2].numel(), (int32_t)nodes, part_size,
                                       &o, &h);
        } else if (kind == 1) {
            o.min_consumers = -1;   // every cache row is materialised, so that workspace row g is upstream's cache row g
            rc = rof_layout_from_v1(p(0), host[1].data_ptr<int32_t>(), p(2), host[2].numel(), p(3),
                                    host[4].data_ptr<int32_t>(), p(5), host[4].numel() - 1, (int32_t)nodes, part_size, &o,
                                    &h);
        } else {
            rc = rof_layout_from_v2(p(0), host[1].data_ptr<int32_t>(), host[2].data_ptr<int32_t>(), p(3),
                                    host[1].numel() - 1, (int32_t)nodes, part_size, &o, &h);
        }
        rof_check(rc, "re-laying out the plan");
        return h;
    }

    // ROF_AUTOTUNE=1 in the environment: how long rows are cut and how the launches are tuned is chosen by timing, as
    // the Python layer's LayoutFamily(autotune=True) does -- the rule's layout against four other cuts on random rows
    // of this width (sum aggregation, HIP events), then rof_layout_calibrate for the launch settings of the winner.
    static bool autotune_wanted() {
        const char *e = getenv("ROF_AUTOTUNE");
        return e && *e && strcmp(e, "0") != 0;
    }

    void autotune(std::unique_ptr<Layout> &lay, const rof_layout_opts &rule_opts, int64_t feat) {
        if (nodes == 0 || feat < 1) return;
        static const int kCuts[][2] = {{128, 32}, {512, 64}, {1024, 128}, {2048, 256}};
        const auto dev = torch::TensorOptions().dtype(torch::kFloat32).device(keep.empty() ? torch::Device(torch::kCUDA) : keep[0].device());
        const int64_t ld = (feat + 3) / 4 * 4;
        torch::Tensor x = torch::randn({nodes, ld}, dev), out = torch::empty({nodes, feat}, dev);
        int64_t st[23];
        rof_check(rof_layout_stats_n(lay->h, st, 23), "reading the layout's counters");
        const int64_t rule_cut = st[20], rule_seg = st[21];
        auto time_of = [&](Layout &l) {
            rof_check(rof_layout_upload(l.h, current_stream()), "uploading the layout");
            const size_t need = rof_layout_workspace_bytes(l.h, (int)feat);
            l.workspace = torch::empty({(int64_t)std::max<size_t>(1, (need + 3) / 4)}, dev);
            float best = 0.f;
            for (int round = 0; round < 3; ++round) {   // the first round warms up
                float ms = 0.f;
                rof_check(rof_aggregate_timed(l.h, x.data_ptr<float>(), ROF_F32, ld, out.data_ptr<float>(), feat, (int)feat, 0,
                                              nullptr, l.workspace.data_ptr(), (size_t)l.workspace.numel() * 4,
                                              current_stream(), 3, &ms),
                          "timing a candidate layout");
                if (round == 1 || (round == 2 && ms < best)) best = ms;
            }
            return best;
        };
        float best_ms = time_of(*lay);
        const float rule_ms = best_ms;
        // other cuts can only matter when some row is long enough to be cut by one of them
        if (st[7] > 0 || st[22] > kCuts[0][0]) {
            for (const auto &c : kCuts) {
                if (c[0] == rule_cut && c[1] == rule_seg) continue;
                rof_layout_opts o = rule_opts;
                o.hub_split = c[0];
                o.segment = c[1];
                std::unique_ptr<Layout> cand(new Layout);
                cand->h = build(o);
                const float ms = time_of(*cand);
                if (ms < 0.99f * rule_ms && ms < best_ms) {   // the rule's choice unless a candidate is measurably faster
                    best_ms = ms;
                    lay = std::move(cand);
                }
            }
        }
        rof_launch_tuning chosen;
        rof_check(rof_layout_calibrate(lay->h, x.data_ptr<float>(), ROF_F32, ld, out.data_ptr<float>(), feat, (int)feat, 0, nullptr,
                                       lay->workspace.data_ptr(), (size_t)lay->workspace.numel() * 4, current_stream(), 2, 3,
                                       &chosen),
                  "calibrating the launch settings");
    }
};

typedef std::vector<int64_t> Key;
std::list<std::pair<Key, std::unique_ptr<Plan>>> g_plans;   // most recently used first
const size_t kMaxPlans = 32;

Plan &plan_of(int kind, int part_size, int64_t nodes, std::vector<torch::Tensor> tensors) {
    Key key{kind, part_size};
    for (const torch::Tensor &t : tensors) {
        TORCH_CHECK(t.scalar_type() == torch::kInt32, "plan tensors must be int32");
        key.push_back((int64_t)(intptr_t)t.data_ptr());
        key.push_back(t.numel());
        key.push_back((int64_t)t._version());
    }
    for (auto it = g_plans.begin(); it != g_plans.end(); ++it)
        if (it->first == key) {
            g_plans.splice(g_plans.begin(), g_plans, it);
            return *g_plans.front().second;
        }
    std::unique_ptr<Plan> p(new Plan);
    p->kind = kind;
    p->part_size = part_size;
    p->nodes = nodes;
    for (const torch::Tensor &t : tensors) p->host.push_back(t.detach().cpu().contiguous());
    p->keep = std::move(tensors);   // the key holds raw addresses: keep their owners alive
    g_plans.emplace_front(std::move(key), std::move(p));
    while (g_plans.size() > kMaxPlans) g_plans.pop_back();
    return *g_plans.front().second;
}

void set_degrees(Layout &lay, const torch::Tensor &degrees, int64_t nodes) {
    TORCH_CHECK(degrees.scalar_type() == torch::kFloat32 && degrees.numel() == nodes,
                "degrees must be a float32 tensor with one entry per node");
    rof_check(rof_layout_upload(lay.h, current_stream()), "uploading the layout");
    if (lay.deg_ptr == degrees.data_ptr() && lay.deg_version == (int64_t)degrees._version()) return;
    rof_check(rof_layout_set_degrees(lay.h, degrees.data_ptr<float>(), current_stream()), "setting the degrees");
    lay.deg_ptr = degrees.data_ptr();
    lay.deg_version = (int64_t)degrees._version();
    lay.deg_keep = degrees;
}

// out[v] = s(v) * sum_u w(u) x[u] over the plan; x may be a column-padded view ([N, feat] with a larger row stride).
// pad_columns: x's rows are allocated up to the next multiple of four floats and the result may keep such rows.
torch::Tensor aggregate(Layout &lay, const torch::Tensor &x, int64_t feat, bool normalized, bool pad_columns, int64_t nodes) {
    TORCH_CHECK(x.dim() == 2 && x.stride(1) == 1 && x.size(0) >= nodes, "x must be a 2-D tensor with one row per node");
    TORCH_CHECK(x.scalar_type() == torch::kFloat32, "x must be float32");
    rof_check(rof_layout_upload(lay.h, current_stream()), "uploading the layout");
    const int64_t padded = (feat + 3) / 4 * 4;
    const bool pad = pad_columns && padded != feat && feat >= 4 && x.stride(0) >= padded;
    torch::Tensor out = pad ? torch::empty({nodes, padded}, x.options()).slice(1, 0, feat) : torch::empty({nodes, feat}, x.options());
    const size_t need = rof_layout_workspace_bytes(lay.h, (int)feat);
    if (!lay.workspace.defined() || (size_t)lay.workspace.numel() * 4 < need || lay.workspace.device() != x.device())
        lay.workspace = torch::empty({(int64_t)std::max<size_t>(1, (need + 3) / 4)}, x.options());
    rof_epilogue ep;
    memset(&ep, 0, sizeof(ep));
    ep.out_dtype = ROF_F32;
    ep.pad_columns = pad ? 1 : 0;
    rof_check(rof_aggregate_epilogue(lay.h, x.data_ptr<float>(), ROF_F32, x.stride(0), out.data_ptr<float>(), out.stride(0),
                                     (int)feat, normalized ? 1 : 0, &ep, lay.workspace.data_ptr(),
                                     (size_t)lay.workspace.numel() * 4, current_stream()),
              "aggregation");
    return out;
}

// tmp = x @ weight (reuse_conv_kernel.cu:302) in rows whose stride is a multiple of four floats, so that they are
// gathered with 16-byte loads; the view returned is [N, out] either way
torch::Tensor update(const torch::Tensor &x, const torch::Tensor &weight) {
    const int64_t f = weight.size(1), pad = (4 - f % 4) % 4;
    if (pad == 0) return torch::mm(x, weight);
    torch::Tensor wpad = torch::cat({weight, weight.new_zeros({weight.size(0), pad})}, 1);
    return torch::mm(x, wpad).slice(1, 0, f);
}

// x^T @ d for tall operands: one GEMM with in * out outputs has too few tiles to fill the GPU, so the rows are cut
// into slabs that form a batched GEMM whose products are added in float32
torch::Tensor weight_grad(const torch::Tensor &x, const torch::Tensor &d) {
    const int64_t n = x.size(0);
    const int64_t slabs = std::min<int64_t>(1024, n / 4096);
    if (slabs < 4) return torch::mm(x.transpose(0, 1), d).to(torch::kFloat32);
    const int64_t m = n / slabs;
    torch::Tensor a = x.slice(0, 0, m * slabs).unflatten(0, {slabs, m});
    torch::Tensor b = d.slice(0, 0, m * slabs).unflatten(0, {slabs, m});
    torch::Tensor out = torch::bmm(a.transpose(1, 2), b).sum(0, false, torch::kFloat32);
    if (m * slabs < n) out += torch::mm(x.slice(0, m * slabs).transpose(0, 1), d.slice(0, m * slabs)).to(torch::kFloat32);
    return out;
}

std::vector<torch::Tensor> forward(Plan &plan, const torch::Tensor &input, const torch::Tensor &weight,
                                   const torch::Tensor &degrees, Layout **used = nullptr) {
    torch::Tensor tmp = update(input, weight);
    Layout &lay = plan.get(weight.size(1));
    set_degrees(lay, degrees, plan.nodes);
    if (used) *used = &lay;
    return {aggregate(lay, tmp, weight.size(1), true, false, plan.nodes)};
}

// upstream aggregates d_output with the same un-transposed plan (reuse_conv_kernel.cu:353-373, 743-808, 1021-1041),
// then the two GEMMs (cu:382-383)
std::vector<torch::Tensor> backward(Plan &plan, const torch::Tensor &d_output, const torch::Tensor &X, const torch::Tensor &W,
                                    const torch::Tensor &degrees, Layout **used = nullptr) {
    const int64_t f = d_output.size(1);
    Layout &lay = plan.get(f);
    set_degrees(lay, degrees, plan.nodes);
    if (used) *used = &lay;
    torch::Tensor d_input_prime = aggregate(lay, d_output, f, true, true, plan.nodes);
    return {torch::mm(d_input_prime, W.transpose(0, 1)), weight_grad(X, d_input_prime)};
}

// upstream's caching kernel leaves the group sums and a ready flag of 1 in the caller's scratch
// (reuse_conv_kernel.cu:476-485)
void fill_cache(Layout &lay, torch::Tensor part_result_cache, int64_t f) {
    const int64_t p = part_result_cache.size(0);
    if (p == 0 || part_result_cache.size(1) != f + 1) return;
    const int64_t ld = (f + 7) / 8 * 8;
    torch::NoGradGuard guard;
    torch::Tensor rows = lay.workspace.slice(0, 0, p * ld).view({p, ld});
    part_result_cache.slice(1, 0, f).copy_(rows.slice(1, 0, f));
    part_result_cache.select(1, f).fill_(1.0);
}

}  // namespace

// reuse_conv.cpp:132-155 (kernel reuse_conv_kernel.cu:123-196): unnormalised sum aggregation of `input` itself
torch::Tensor SAG(torch::Tensor input, torch::Tensor row_pointers, torch::Tensor column_index, torch::Tensor degrees,
                  torch::Tensor part_pointers, torch::Tensor part2Node, int partSize, int dimWorker, int warpPerBlock) {
    CHECK_INPUT(input);
    CHECK_INPUT(row_pointers);
    CHECK_INPUT(column_index);
    CHECK_INPUT(degrees);
    CHECK_INPUT(part_pointers);
    CHECK_INPUT(part2Node);
    Plan &plan = plan_of(0, partSize, input.size(0), {column_index, part_pointers, part2Node});
    return aggregate(plan.get(input.size(1)), input, input.size(1), false, false, plan.nodes);
}

// reuse_conv.cpp:158-176
std::vector<torch::Tensor> GNNA_forward(torch::Tensor input, torch::Tensor weight, torch::Tensor column_index,
                                        torch::Tensor degrees, torch::Tensor part_pointers, torch::Tensor part2Node,
                                        int partSize, int dimWorker, int warpPerBlock) {
    CHECK_INPUT(input);
    CHECK_INPUT(weight);
    CHECK_INPUT(column_index);
    CHECK_INPUT(degrees);
    CHECK_INPUT(part_pointers);
    CHECK_INPUT(part2Node);
    return forward(plan_of(0, partSize, input.size(0), {column_index, part_pointers, part2Node}), input, weight, degrees);
}

// reuse_conv.cpp:179-196
std::vector<torch::Tensor> GNNA_backward(torch::Tensor d_output, torch::Tensor X, torch::Tensor W, torch::Tensor column_index,
                                         torch::Tensor degrees, torch::Tensor part_pointers, torch::Tensor part2Node,
                                         int partSize, int dimWorker, int warpPerBlock) {
    CHECK_INPUT(d_output);
    CHECK_INPUT(X);
    CHECK_INPUT(W);
    CHECK_INPUT(column_index);
    CHECK_INPUT(degrees);
    CHECK_INPUT(part_pointers);
    CHECK_INPUT(part2Node);
    return backward(plan_of(0, partSize, X.size(0), {column_index, part_pointers, part2Node}), d_output, X, W, degrees);
}

// reuse_conv.cpp:199-240
std::vector<torch::Tensor> reuse_spmm_forward_v1(torch::Tensor input, torch::Tensor weight, torch::Tensor column_index,
                                                 torch::Tensor degrees, torch::Tensor part_pointers, torch::Tensor part2Node,
                                                 int partSize, int dimWorker, int warpPerBlock,
                                                 torch::Tensor part_result_cache, torch::Tensor part_cache_flagindex,
                                                 torch::Tensor part_pointers_cache, torch::Tensor column_index_cache) {
    CHECK_INPUT(input);
    CHECK_INPUT(weight);
    CHECK_INPUT(column_index);
    CHECK_INPUT(degrees);
    CHECK_INPUT(part_pointers);
    CHECK_INPUT(part2Node);
    CHECK_INPUT(part_result_cache);
    CHECK_INPUT(part_cache_flagindex);
    CHECK_INPUT(part_pointers_cache);
    CHECK_INPUT(column_index_cache);
    Plan &plan = plan_of(1, partSize, input.size(0),
                         {column_index, part_pointers, part2Node, part_cache_flagindex, part_pointers_cache, column_index_cache});
    Layout *lay = nullptr;
    std::vector<torch::Tensor> out = forward(plan, input, weight, degrees, &lay);
    fill_cache(*lay, part_result_cache, weight.size(1));
    return out;
}

// reuse_conv.cpp:243-285
std::vector<torch::Tensor> reuse_spmm_backward_v1(torch::Tensor d_output, torch::Tensor X, torch::Tensor W,
                                                  torch::Tensor column_index, torch::Tensor degrees, torch::Tensor part_pointers,
                                                  torch::Tensor part2Node, int partSize, int dimWorker, int warpPerBlock,
                                                  torch::Tensor part_result_cache, torch::Tensor part_cache_flagindex,
                                                  torch::Tensor part_pointers_cache, torch::Tensor column_index_cache) {
    CHECK_INPUT(d_output);
    CHECK_INPUT(X);
    CHECK_INPUT(W);
    CHECK_INPUT(column_index);
    CHECK_INPUT(degrees);
    CHECK_INPUT(part_pointers);
    CHECK_INPUT(part2Node);
    CHECK_INPUT(part_result_cache);
    CHECK_INPUT(part_cache_flagindex);
    CHECK_INPUT(part_pointers_cache);
    CHECK_INPUT(column_index_cache);
    Plan &plan = plan_of(1, partSize, X.size(0),
                         {column_index, part_pointers, part2Node, part_cache_flagindex, part_pointers_cache, column_index_cache});
    Layout *lay = nullptr;
    std::vector<torch::Tensor> res = backward(plan, d_output, X, W, degrees, &lay);
    fill_cache(*lay, part_result_cache, d_output.size(1));
    return res;
}

// reuse_conv.cpp:288-314
std::vector<torch::Tensor> reuse_spmm_forward_v2(torch::Tensor input, torch::Tensor weight, torch::Tensor uniqpart_column_index,
                                                 torch::Tensor degrees, torch::Tensor uniqpart_pointers,
                                                 torch::Tensor part2Node_ptr, torch::Tensor part2Node_col, int partSize,
                                                 int dimWorker, int warpPerBlock) {
    CHECK_INPUT(input);
    CHECK_INPUT(weight);
    CHECK_INPUT(uniqpart_column_index);
    CHECK_INPUT(degrees);
    CHECK_INPUT(uniqpart_pointers);
    CHECK_INPUT(part2Node_ptr);
    CHECK_INPUT(part2Node_col);
    return forward(plan_of(2, partSize, input.size(0), {uniqpart_column_index, uniqpart_pointers, part2Node_ptr, part2Node_col}),
                   input, weight, degrees);
}

// reuse_conv.cpp:317-346
std::vector<torch::Tensor> reuse_spmm_backward_v2(torch::Tensor d_output, torch::Tensor X, torch::Tensor W,
                                                  torch::Tensor uniqpart_column_index, torch::Tensor degrees,
                                                  torch::Tensor uniqpart_pointers, torch::Tensor part2Node_ptr,
                                                  torch::Tensor part2Node_col, int partSize, int dimWorker, int warpPerBlock) {
    CHECK_INPUT(d_output);
    CHECK_INPUT(X);
    CHECK_INPUT(W);
    CHECK_INPUT(uniqpart_column_index);
    CHECK_INPUT(degrees);
    CHECK_INPUT(uniqpart_pointers);
    CHECK_INPUT(part2Node_ptr);
    CHECK_INPUT(part2Node_col);
    return backward(plan_of(2, partSize, X.size(0), {uniqpart_column_index, uniqpart_pointers, part2Node_ptr, part2Node_col}),
                    d_output, X, W, degrees);
}

void clear_layout_cache() { g_plans.clear(); }

// the module list of reuse_conv.cpp:353-365, plus the cache control
PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.def("SAG", &SAG, "unnormalised sum aggregation (gfx950)");
    m.def("GNNA_forward", &GNNA_forward, "GCN layer forward without reuse (gfx950)");
    m.def("GNNA_backward", &GNNA_backward, "GCN layer backward without reuse (gfx950)");
    m.def("reuse_forward_v1", &reuse_spmm_forward_v1, "GCN layer forward, v1 plan tensors (gfx950)");
    m.def("reuse_backward_v1", &reuse_spmm_backward_v1, "GCN layer backward, v1 plan tensors (gfx950)");
    m.def("reuse_forward_v2", &reuse_spmm_forward_v2, "GCN layer forward, v2 plan tensors (gfx950)");
    m.def("reuse_backward_v2", &reuse_spmm_backward_v2, "GCN layer backward, v2 plan tensors (gfx950)");
    m.def("clear_layout_cache", &clear_layout_cache, "drop the device layouts cached per plan");
}
