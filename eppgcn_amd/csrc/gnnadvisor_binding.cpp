// Python extension module `GNNAdvisor` for PyTorch-ROCm: the twelve functions the
// reference's Python calls (EPPGCN/GCNConv/EPPGCN.cpp:388-403), same positional
// signatures, implemented over the C ABI of libeppgcn_hip.so.  torch supplies the
// tensors and the current HIP stream (and torch::mm for dense products whose shapes
// the library's tall-and-skinny kernels do not cover); everything else happens in
// the HIP library.  Host C++ only: no device code in this file.
//
// Differences from the reference binding, all deliberate:
//   - errors raise (RuntimeError in Python) instead of printf + exit(-1);
//   - work is issued on torch's current stream and is asynchronous unless a host
//     value is returned;
//   - build_part computes on the device and returns int32 tensors (the reference
//     loops on the CPU and returns float32, which corrupts offsets above 2^24);
//   - compact_back_edge's info tensor is float64 so that int(info[0].item()) is
//     exact for any edge count;
//   - split_back_part's part_pointer has num_edges + 1 entries, so the terminator
//     is always in bounds;
//   - get_map_back_part_size never returns less than 1: where the fitted regression drops below 1
//     (large paths) it returns the group size of the rule fitted for the wave64 kernels;
//   - get_ginfo also accepts a CPU tensor, as the reference's host loop does;
//   - the module keeps, per group array it has seen, a column-blocked execution plan for the
//     aggregation kernels (built on first use, about 4 bytes per edge, the 8 most recently used
//     kept); it affects speed only.
#include <torch/extension.h>

#include <c10/hip/HIPStream.h>

#include <cstdint>
#include <list>
#include <vector>

#include "eppgcn_hip.h"

namespace {

using torch::Tensor;

void check(int rc, const char* what)
{
    TORCH_CHECK(rc == 0, what, " failed (", rc, "): ", eppgcn_last_error());
}

#define CHECK_DEVICE(x) TORCH_CHECK((x).is_cuda(), #x " must be a GPU tensor")
#define CHECK_CONTIGUOUS(x) TORCH_CHECK((x).is_contiguous(), #x " must be contiguous")
#define CHECK_INPUT(x) \
    CHECK_DEVICE(x);   \
    CHECK_CONTIGUOUS(x)
#define CHECK_I32(x) \
    CHECK_INPUT(x);  \
    TORCH_CHECK((x).scalar_type() == torch::kInt32, #x " must be int32")
#define CHECK_F32(x) \
    CHECK_INPUT(x);  \
    TORCH_CHECK((x).scalar_type() == torch::kFloat32, #x " must be float32")
#define CHECK_MASK(x) \
    CHECK_INPUT(x);   \
    TORCH_CHECK((x).scalar_type() == torch::kBool || (x).scalar_type() == torch::kUInt8, #x " must be bool")

// Slots and vertices are int32 on the device, and the kernels step through slot ranges in strides of
// up to 1024 past a group's end before clamping: leave that much headroom below 2^31.
#define CHECK_COUNTS(edges, vertices)                                                                      \
    TORCH_CHECK((edges).numel() <= INT32_MAX - 1024, #edges " holds more slots than int32 indexing allows"); \
    TORCH_CHECK((vertices) <= INT32_MAX - 1024, "more vertices than int32 indexing allows")

void* stream_of(const Tensor& t)
{
    return static_cast<void*>(c10::hip::getCurrentHIPStream(t.get_device()).stream());
}

const int32_t* i32(const Tensor& t) { return t.numel() ? t.data_ptr<int32_t>() : nullptr; }
const float* f32(const Tensor& t) { return t.numel() ? t.data_ptr<float>() : nullptr; }

Tensor workspace(size_t bytes, const Tensor& like)
{
    return torch::empty({static_cast<int64_t>((bytes + 7) / 8)}, like.options().dtype(torch::kInt64));
}

// ---------------------------------------------------------------- plan cache
// The column-blocked execution plan depends only on the groups and the column ids, which a
// training run passes unchanged every epoch.  Entries are keyed by storage address, length,
// tensor version and block-size class, and hold references to the key tensors so that an
// address cannot be reused for other data while its entry lives.
// Staleness rule: an entry is invalidated by writes that bump torch's version counter (ordinary
// in-place tensor operations).  A writer that bypasses the counter - `.data` / detach() in-place
// operations, a raw-pointer kernel of another extension, this library's own C ABI writing into the
// same storage - leaves the cached plan describing the old groups; after such a write call
// clear_plans() before the next layer operation.
struct PlanEntry {
    const void* part_ptr;
    const void* col;
    const void* rows;
    int64_t num_parts;
    int64_t num_nodes;          // the plan's layout depends on it
    int64_t version_part, version_col, version_rows;
    int dim_class;
    Tensor keep_part, keep_col, keep_rows, plan;
    const void* plan_ptr;
};
std::list<PlanEntry> g_plans;
constexpr size_t kMaxPlans = 8;
// An entry that leaves the cache gives its plan's memory back to torch: the library is told first, so that it
// forgets the header it read at that address.
void drop_oldest_plan()
{
    eppgcn_plan_release(g_plans.back().plan_ptr);
    g_plans.pop_back();
}
void drop_all_plans()
{
    for (const PlanEntry& e : g_plans) eppgcn_plan_release(e.plan_ptr);
    g_plans.clear();
}
int g_plan_policy = 0;   // 0: where eppgcn_plan_recommended says so, 1: always, -1: never

int dim_class_of(int dim) { return dim <= 32 ? 0 : dim <= 128 ? 1 : 2; }
int dim_of_class(int c) { return c == 0 ? 32 : c == 1 ? 128 : 256; }

Tensor aligned_bytes(size_t bytes, const Tensor& like, void** base)
{
    auto t = torch::empty({static_cast<int64_t>(bytes + 256)}, like.options().dtype(torch::kUInt8));
    *base = reinterpret_cast<void*>((reinterpret_cast<uintptr_t>(t.data_ptr()) + 255) / 256 * 256);
    return t;
}

// rows: part2Node (forward groups, is_forward) or the per-edge id list (backward path);
// num_slots < 0: read it from part_ptr[num_parts] when the plan has to be built
const void* plan_for(const Tensor& part_ptr, const Tensor& col, const Tensor& rows, bool is_forward, int64_t num_parts,
                     int64_t num_slots, int num_nodes, int dim, int block_shift = 0)
{
    if (num_parts <= 0 || g_plan_policy < 0) return nullptr;
    if (g_plan_policy == 0 && !eppgcn_plan_recommended(num_nodes, dim)) return nullptr;
    const int dc = dim_class_of(dim);
    for (auto it = g_plans.begin(); it != g_plans.end(); ++it) {
        if (it->part_ptr == part_ptr.data_ptr() && it->col == col.data_ptr() && it->rows == rows.data_ptr() &&
            it->num_parts == num_parts && it->num_nodes == num_nodes && it->dim_class == dc &&
            it->version_part == static_cast<int64_t>(part_ptr._version()) &&
            it->version_col == static_cast<int64_t>(col._version()) &&
            it->version_rows == static_cast<int64_t>(rows._version())) {
            g_plans.splice(g_plans.begin(), g_plans, it);   // most recently used first
            return g_plans.front().plan_ptr;
        }
    }
    if (num_slots < 0) num_slots = part_ptr[num_parts].item<int64_t>();   // slots the groups cover (one 4-byte read)
    PlanEntry e{part_ptr.data_ptr(), col.data_ptr(), rows.data_ptr(), num_parts, num_nodes,
                static_cast<int64_t>(part_ptr._version()), static_cast<int64_t>(col._version()),
                static_cast<int64_t>(rows._version()), dc, part_ptr, col, rows, Tensor(), nullptr};
    const size_t bytes = eppgcn_plan_bytes(num_parts, num_slots, num_nodes);
    void* base = nullptr;
    e.plan = aligned_bytes(bytes, part_ptr, &base);
    e.plan_ptr = base;
    const size_t wbytes = eppgcn_plan_workspace_bytes(num_parts, num_slots);
    void* wbase = nullptr;
    auto ws = aligned_bytes(wbytes, part_ptr, &wbase);
    check(eppgcn_build_plan(part_ptr.data_ptr<int32_t>(), col.data_ptr<int32_t>(),
                            is_forward ? rows.data_ptr<int32_t>() : nullptr,
                            is_forward ? nullptr : rows.data_ptr<int32_t>(), static_cast<int>(num_parts), num_slots,
                            num_nodes, dim_of_class(dc), block_shift, base, bytes, wbase, wbytes, stream_of(part_ptr)),
          "build_plan");
    // once per group array: wait for the build, refuse a plan whose look-back scan stalled and let the
    // library read the counts of the plan's stream form
    check(eppgcn_plan_status(base, static_cast<int>(num_parts), num_slots, num_nodes, nullptr, stream_of(part_ptr)),
          "build_plan");
    g_plans.push_front(std::move(e));
    if (g_plans.size() > kMaxPlans) drop_oldest_plan();
    return g_plans.front().plan_ptr;
}

// Per backward path, remembered from its first use:
//   - whether its plan is column-blocked: a heavily pruned path gathers from few distinct rows, which
//     stay cached in any order, so only paths that keep at least half of the edges are blocked;
//   - the bitmap of the rows it gathers, when they are fewer than half of the vertices: the
//     pre-scaling pass of the gradient then touches those rows only.
// An entry is valid for exactly the tensors it was made from (same storage, same version counters);
// it holds references to them so that their memory cannot be handed to other tensors meanwhile.
struct PathChoice {
    const void* part_ptr;
    const void* edge_ptr;
    int64_t num_parts, num_nodes;
    int64_t version_part, version_edge;
    bool use_plan;
    Tensor keep_part, keep_edge, gathered;     // gathered: undefined when the path reads most rows
};
std::list<PathChoice> g_path_choices;

const PathChoice& path_choice(const Tensor& part_pointer, const Tensor& edge_list, int64_t num_parts, int num_nodes,
                              int64_t* valid_len_out)
{
    *valid_len_out = -1;
    for (auto it = g_path_choices.begin(); it != g_path_choices.end(); ++it) {
        if (it->part_ptr == part_pointer.data_ptr() && it->edge_ptr == edge_list.data_ptr() &&
            it->num_parts == num_parts && it->num_nodes == num_nodes &&
            it->version_part == static_cast<int64_t>(part_pointer._version()) &&
            it->version_edge == static_cast<int64_t>(edge_list._version())) {
            g_path_choices.splice(g_path_choices.begin(), g_path_choices, it);
            return g_path_choices.front();
        }
    }
    const int64_t valid_len = part_pointer[num_parts].item<int64_t>();
    *valid_len_out = valid_len;
    TORCH_CHECK(valid_len >= 0 && valid_len <= edge_list.numel(), "partPointer[numParts] lies outside edgeList");
    PathChoice c{part_pointer.data_ptr(), edge_list.data_ptr(), num_parts, num_nodes,
                 static_cast<int64_t>(part_pointer._version()), static_cast<int64_t>(edge_list._version()),
                 g_plan_policy > 0 || 2 * valid_len >= edge_list.numel(), part_pointer, edge_list, Tensor()};
    auto bitmap = torch::empty({(static_cast<int64_t>(num_nodes) + 31) / 32 + 1}, edge_list.options());
    int64_t distinct = 0;
    check(eppgcn_mark_gathered_rows(i32(edge_list), valid_len, num_nodes,
                                    reinterpret_cast<uint32_t*>(bitmap.data_ptr<int32_t>()),
                                    bitmap.data_ptr<int32_t>() + bitmap.numel() - 1, &distinct, stream_of(edge_list)),
          "mark_gathered_rows");
    if (2 * distinct < num_nodes) c.gathered = bitmap;
    g_path_choices.push_front(std::move(c));
    if (g_path_choices.size() > 8) g_path_choices.pop_back();
    return g_path_choices.front();
}

// room for the pre-scaled table and, behind it, the partial sums of a call through the plan's stream form
Tensor feature_scratch(const Tensor& feats, const void* plan)
{
    const size_t n = eppgcn_plan_workspace_floats(plan, feats.size(0), static_cast<int>(feats.size(1)));
    return torch::empty({static_cast<int64_t>(n)}, feats.options());
}

// ---------------------------------------------------------------- dense update helpers
// The three products around the aggregation run in the library's tall-and-skinny kernels when the
// shapes fit them (eppgcn_update_supported) and in torch::mm otherwise; g_dense_policy -1 forces mm.
int g_dense_policy = 0;

int dense_support(const Tensor& X, const Tensor& W)
{
    if (g_dense_policy < 0) return 0;
    return eppgcn_update_supported(static_cast<int>(X.size(1)), static_cast<int>(W.size(1)));
}

// scale[r] * act(X) * W as the padded, pre-scaled feature table the aggregation gathers from
Tensor scaled_product(const Tensor& X, const Tensor& W, const Tensor& degrees, bool relu_input, const void* plan,
                      size_t* ws_floats)
{
    const int64_t n = X.size(0);
    const int dim = static_cast<int>(W.size(1));
    *ws_floats = eppgcn_plan_workspace_floats(plan, n, dim);
    auto scaled = torch::empty({static_cast<int64_t>(*ws_floats)}, X.options());
    check(eppgcn_update_forward_table(scaled.data_ptr<float>(), *ws_floats, X.data_ptr<float>(), W.data_ptr<float>(), f32(degrees),
                                      relu_input ? 1 : 0, n, static_cast<int>(X.size(1)), dim, stream_of(X)),
          "update_forward_table");
    return scaled;
}

// g_masked_update: 1 (default) lets the pruned backward hand the bitmap of the rows it wrote to the dense products
// (rows outside the path are then neither cleared nor read); 0 clears and reads every row.
int g_masked_update = 1;

// {dX or an empty tensor, dW} from the aggregated gradient G; `rows`: nullptr, or the bitmap of the rows of G that
// are defined (the others count as zeros and are not read)
std::vector<Tensor> dense_backward(const Tensor& G, const Tensor& X, const Tensor& W, bool need_dx, bool relu_input,
                                   const uint32_t* rows = nullptr)
{
    const int64_t n = X.size(0);
    const int in_dim = static_cast<int>(X.size(1)), out_dim = static_cast<int>(W.size(1));
    const int sup = dense_support(X, W);
    Tensor d_weight, d_input;
    if (rows) {
        // only reached when the shapes fit the library's kernels (the caller checked dense_support)
        d_weight = torch::empty({in_dim, out_dim}, X.options());
        d_input = need_dx ? torch::empty({n, in_dim}, X.options()) : torch::empty({0}, X.options());
        const size_t nbytes = eppgcn_update_workspace_bytes(n, in_dim, out_dim);
        auto ws = torch::empty({static_cast<int64_t>((nbytes + 3) / 4) + 1}, X.options());
        check(eppgcn_update_backward_rows(need_dx ? d_input.data_ptr<float>() : nullptr, d_weight.data_ptr<float>(), f32(X),
                                          f32(G), f32(W), relu_input ? 1 : 0, rows, n, in_dim, out_dim,
                                          ws.data_ptr<float>(), nbytes, stream_of(X)),
              "update_backward_rows");
        return {d_input, d_weight};
    }
    if (need_dx && (sup & 6) == 6) {
        // both gradients from one call: narrow layers read X and G once for the two products
        d_weight = torch::empty({in_dim, out_dim}, X.options());
        d_input = torch::empty({n, in_dim}, X.options());
        const size_t nbytes = eppgcn_update_workspace_bytes(n, in_dim, out_dim);
        auto ws = torch::empty({static_cast<int64_t>((nbytes + 3) / 4) + 1}, X.options());
        check(eppgcn_update_backward(d_input.data_ptr<float>(), d_weight.data_ptr<float>(), f32(X), f32(G), f32(W),
                                     relu_input ? 1 : 0, n, in_dim, out_dim, ws.data_ptr<float>(), nbytes, stream_of(X)),
              "update_backward");
        return {d_input, d_weight};
    }
    if (sup & 4) {
        d_weight = torch::empty({in_dim, out_dim}, X.options());
        const size_t nbytes = eppgcn_update_workspace_bytes(n, in_dim, out_dim);
        auto ws = torch::empty({static_cast<int64_t>((nbytes + 3) / 4) + 1}, X.options());
        check(eppgcn_update_backward_weight(d_weight.data_ptr<float>(), f32(X), f32(G), relu_input ? 1 : 0, n, in_dim,
                                            out_dim, ws.data_ptr<float>(), nbytes, stream_of(X)),
              "update_backward_weight");
    } else {
        d_weight = torch::mm((relu_input ? torch::relu(X) : X).transpose(0, 1), G);
    }
    if (!need_dx) {
        d_input = torch::empty({0}, X.options());
    } else if (sup & 2) {
        d_input = torch::empty({n, in_dim}, X.options());
        check(eppgcn_update_backward_input(d_input.data_ptr<float>(), f32(G), f32(W), relu_input ? f32(X) : nullptr, n,
                                           in_dim, out_dim, stream_of(X)),
              "update_backward_input");
    } else {
        d_input = torch::mm(G, W.transpose(0, 1));
        if (relu_input) d_input = d_input * (X > 0);
    }
    return {d_input, d_weight};
}

// ---------------------------------------------------------------- forward / backward
std::vector<Tensor> forward(Tensor input, Tensor weight, Tensor row_pointers, Tensor column_index, Tensor degrees,
                            Tensor part_pointers, Tensor part2Node, int partSize, int dimWorker, int warpPerBlock,
                            bool relu_input)
{
    CHECK_F32(input); CHECK_F32(weight); CHECK_I32(row_pointers); CHECK_I32(column_index);
    CHECK_F32(degrees); CHECK_I32(part_pointers); CHECK_I32(part2Node);
    TORCH_CHECK(input.dim() == 2 && weight.dim() == 2 && input.size(1) == weight.size(0), "shape mismatch");
    TORCH_CHECK(degrees.numel() == input.size(0), "degrees must have one entry per vertex");
    TORCH_CHECK(part_pointers.numel() >= part2Node.numel() + 1, "part_pointers needs num_parts + 1 entries");
    CHECK_COUNTS(column_index, input.size(0));
    const int64_t n = input.size(0);
    const int dim = static_cast<int>(weight.size(1));
    auto output = torch::empty({n, dim}, input.options());
    const void* plan = plan_for(part_pointers, column_index, part2Node, true, part2Node.numel(), column_index.numel(),
                                static_cast<int>(n), dim);
    if (n > 0 && (dense_support(input, weight) & 1)) {
        // the product is written scaled and padded, ready to be gathered: no separate scaling pass
        size_t ws_floats = 0;
        auto scaled = scaled_product(input, weight, degrees, relu_input, plan, &ws_floats);
        check(eppgcn_spmm_forward(output.data_ptr<float>(), nullptr, i32(row_pointers), i32(column_index),
                                  f32(degrees), i32(part_pointers), i32(part2Node), static_cast<int>(n), dim,
                                  static_cast<int>(part2Node.numel()), partSize, dimWorker, warpPerBlock,
                                  scaled.data_ptr<float>(), ws_floats, plan, stream_of(input)),
              "forward");
        return {output};
    }
    auto tmp = torch::mm(relu_input ? torch::relu(input) : input, weight);
    // tmp is ours: when its rows need no padding and no partial sums follow the table it is scaled in place,
    // otherwise into scratch
    const size_t ws_floats = eppgcn_plan_workspace_floats(plan, tmp.size(0), dim);
    auto scaled = ws_floats == static_cast<size_t>(tmp.numel())
                      ? tmp
                      : torch::empty({static_cast<int64_t>(ws_floats)}, tmp.options());
    check(eppgcn_spmm_forward(output.data_ptr<float>(), f32(tmp), i32(row_pointers), i32(column_index),
                              f32(degrees), i32(part_pointers), i32(part2Node), static_cast<int>(n), dim,
                              static_cast<int>(part2Node.numel()), partSize, dimWorker, warpPerBlock,
                              scaled.numel() ? scaled.data_ptr<float>() : nullptr, ws_floats, plan, stream_of(input)),
          "forward");
    return {output};
}

std::vector<Tensor> backward(Tensor d_output, Tensor X, Tensor W, Tensor row_pointers, Tensor column_index,
                             Tensor degrees, Tensor part_pointers, Tensor part2Node, int partSize, int dimWorker,
                             int warpPerBlock, bool need_dx, bool relu_input)
{
    CHECK_F32(d_output); CHECK_F32(X); CHECK_F32(W); CHECK_I32(row_pointers); CHECK_I32(column_index);
    CHECK_F32(degrees); CHECK_I32(part_pointers); CHECK_I32(part2Node);
    TORCH_CHECK(d_output.dim() == 2 && degrees.numel() == d_output.size(0), "shape mismatch");
    TORCH_CHECK(X.dim() == 2 && W.dim() == 2 && X.size(0) == d_output.size(0) && X.size(1) == W.size(0) &&
                    W.size(1) == d_output.size(1), "X, W and d_output do not fit together");
    TORCH_CHECK(part_pointers.numel() >= part2Node.numel() + 1, "part_pointers needs num_parts + 1 entries");
    CHECK_COUNTS(column_index, d_output.size(0));
    auto d_input_prime = torch::empty_like(d_output);
    const void* plan = plan_for(part_pointers, column_index, part2Node, true, part2Node.numel(), column_index.numel(),
                                static_cast<int>(d_output.size(0)), static_cast<int>(d_output.size(1)));
    auto scaled = feature_scratch(d_output, plan);     // d_output belongs to autograd: scale into scratch
    check(eppgcn_spmm_backward(d_input_prime.data_ptr<float>(), f32(d_output), i32(row_pointers),
                               i32(column_index), f32(degrees), i32(part_pointers), i32(part2Node),
                               static_cast<int>(d_output.size(0)), static_cast<int>(d_output.size(1)),
                               static_cast<int>(part2Node.numel()), partSize, dimWorker, warpPerBlock,
                               scaled.numel() ? scaled.data_ptr<float>() : nullptr, static_cast<size_t>(scaled.numel()),
                               plan, stream_of(d_output)),
          "backward");
    return dense_backward(d_input_prime, X, W, need_dx, relu_input);
}

void mask_forward(Tensor id, Tensor partPointer, Tensor edgeList, Tensor src_mask, Tensor ngh_mask,
                  Tensor backEdgeMask, Tensor node_degs, int num_layers, int layer, int blockx, int blocky)
{
    CHECK_I32(id); CHECK_I32(partPointer); CHECK_I32(edgeList); CHECK_MASK(src_mask); CHECK_MASK(ngh_mask);
    CHECK_I32(backEdgeMask); CHECK_I32(node_degs);
    const bool is_last = layer == num_layers;
    TORCH_CHECK(partPointer.numel() >= id.numel() + 1, "partPointer needs num_parts + 1 entries");
    TORCH_CHECK(backEdgeMask.numel() >= edgeList.numel(), "backEdgeMask is shorter than the edge list");
    TORCH_CHECK(src_mask.numel() == node_degs.numel(), "src_mask and node_degs must have one entry per vertex");
    CHECK_COUNTS(edgeList, node_degs.numel());
    TORCH_CHECK(is_last || ngh_mask.numel() == node_degs.numel(), "ngh_mask must have one entry per vertex");
    check(eppgcn_mask_forward(i32(id), i32(partPointer), i32(edgeList),
                              static_cast<const uint8_t*>(src_mask.data_ptr()),
                              ngh_mask.numel() ? static_cast<uint8_t*>(ngh_mask.data_ptr()) : nullptr,
                              backEdgeMask.data_ptr<int32_t>(), node_degs.data_ptr<int32_t>(),
                              static_cast<int>(id.numel()), edgeList.numel(), is_last ? 1 : 0, blockx, blocky,
                              stream_of(id)),
          "mask_forward");
}

std::vector<Tensor> ours_backward(Tensor d_output, Tensor X, Tensor W, Tensor id, Tensor partPointer, Tensor edgeList,
                                  Tensor degrees, int partSize, int numParts, int layer, int blockx, int blocky,
                                  bool need_dx, bool relu_input)
{
    CHECK_F32(d_output); CHECK_F32(X); CHECK_F32(W); CHECK_I32(id); CHECK_I32(partPointer); CHECK_I32(edgeList);
    CHECK_F32(degrees);
    TORCH_CHECK(d_output.dim() == 2 && degrees.numel() == d_output.size(0), "shape mismatch");
    TORCH_CHECK(X.dim() == 2 && W.dim() == 2 && X.size(0) == d_output.size(0) && X.size(1) == W.size(0) &&
                    W.size(1) == d_output.size(1), "X, W and d_output do not fit together");
    TORCH_CHECK(numParts >= 0 && partPointer.numel() >= static_cast<int64_t>(numParts) + 1,
                "partPointer needs numParts + 1 entries");
    CHECK_COUNTS(edgeList, d_output.size(0));
    auto d_input_prime = torch::empty_like(d_output);
    const int num_nodes = static_cast<int>(d_output.size(0));
    const void* plan = nullptr;
    const uint32_t* gathered = nullptr;
    if (numParts > 0) {
        int64_t valid_len = -1;
        const PathChoice& choice = path_choice(partPointer, edgeList, numParts, num_nodes, &valid_len);
        if (choice.gathered.defined())
            gathered = reinterpret_cast<const uint32_t*>(choice.gathered.data_ptr<int32_t>());
        // a heavily pruned path keeps its groups in one block (its few gathered rows stay cached anyway)
        plan = plan_for(partPointer, edgeList, id, false, numParts, valid_len, num_nodes,
                        static_cast<int>(d_output.size(1)), choice.use_plan ? 0 : 31);
    }
    auto scaled = feature_scratch(d_output, plan);     // d_output belongs to autograd: scale into scratch
    // The aggregated gradient is only read by the two dense products below.  When they run in the library's kernels
    // (which take the bitmap of the rows the aggregation wrote), the rows outside the path are neither cleared
    // nor read - the row-masked products the reference sketches in its comments (EPPGCN_kernel.cu:607,616).
    const int sup = dense_support(X, W);
    const bool masked = g_masked_update > 0 && plan && (sup & 4) && (!need_dx || (sup & 2));
    const uint32_t* written = nullptr;
    if (masked) {
        check(eppgcn_ours_backward_rows(d_input_prime.data_ptr<float>(), f32(d_output), i32(id), i32(partPointer),
                                        i32(edgeList), f32(degrees), static_cast<int>(d_output.size(0)),
                                        static_cast<int>(d_output.size(1)), numParts, partSize > 0 ? partSize : 1, layer,
                                        blockx, blocky, scaled.numel() ? scaled.data_ptr<float>() : nullptr,
                                        static_cast<size_t>(scaled.numel()), plan, gathered, &written, nullptr,
                                        stream_of(d_output)),
              "ours_backward_rows");
    } else {
        check(eppgcn_ours_backward(d_input_prime.data_ptr<float>(), f32(d_output), i32(id), i32(partPointer),
                                   i32(edgeList), f32(degrees), static_cast<int>(d_output.size(0)),
                                   static_cast<int>(d_output.size(1)), numParts, partSize > 0 ? partSize : 1, layer, blockx,
                                   blocky, scaled.numel() ? scaled.data_ptr<float>() : nullptr,
                                   static_cast<size_t>(scaled.numel()), plan, gathered, stream_of(d_output)),
              "ours_backward");
    }
    return dense_backward(d_input_prime, X, W, need_dx, relu_input, written);
}

// ---------------------------------------------------------------- path preparation
std::vector<Tensor> build_part(int partSize, Tensor indptr)
{
    TORCH_CHECK(partSize >= 1, "partSize must be >= 1");
    TORCH_CHECK(indptr.scalar_type() == torch::kInt32 && indptr.dim() == 1 && indptr.numel() >= 1,
                "indptr must be a 1-D int32 tensor");
    auto dptr = indptr.is_cuda() ? indptr.contiguous() : indptr.contiguous().to(torch::kCUDA);
    const int num_nodes = static_cast<int>(dptr.numel() - 1);
    const int64_t num_edges = (dptr[num_nodes] - dptr[0]).item<int64_t>();
    const int64_t capacity = num_edges / partSize + num_nodes + 1;
    auto part_ptr = torch::empty({capacity}, dptr.options());
    auto part2node = torch::empty({capacity > 1 ? capacity - 1 : 1}, dptr.options());
    const size_t bytes = eppgcn_split_workspace_bytes(num_nodes);
    auto ws = workspace(bytes, dptr);
    int64_t num_parts = 0;
    check(eppgcn_build_part(dptr.data_ptr<int32_t>(), num_nodes, partSize, part_ptr.data_ptr<int32_t>(),
                            part2node.data_ptr<int32_t>(), capacity, ws.data_ptr(), bytes, nullptr, &num_parts,
                            stream_of(dptr)),
          "build_part");
    return {part_ptr.narrow(0, 0, num_parts + 1), part2node.narrow(0, 0, num_parts)};
}

struct Compacted {
    Tensor id, edge_list;
    int64_t valid_len;
};

Compacted compact(const Tensor& edge_mask, const Tensor& column_index)
{
    CHECK_I32(edge_mask); CHECK_I32(column_index);
    TORCH_CHECK(column_index.numel() >= edge_mask.numel(), "column_index is shorter than edge_mask");
    const int64_t length = edge_mask.numel();
    Compacted c{torch::empty_like(edge_mask), torch::empty({length}, column_index.options()), 0};
    const size_t bytes = eppgcn_compact_workspace_bytes(length);
    auto ws = workspace(bytes, edge_mask);
    check(eppgcn_compact_back_edge(i32(edge_mask), i32(column_index), c.id.data_ptr<int32_t>(),
                                   c.edge_list.data_ptr<int32_t>(), length, ws.data_ptr(), bytes, nullptr,
                                   &c.valid_len, stream_of(edge_mask)),
          "compact_back_edge");
    return c;
}

int64_t valid_nodes(const Tensor& node_deg)
{
    CHECK_I32(node_deg);
    auto d = torch::empty({1}, node_deg.options());
    int64_t v = 0;
    check(eppgcn_count_nonzero(i32(node_deg), node_deg.numel(), d.data_ptr<int32_t>(), &v, stream_of(node_deg)),
          "count_nonzero");
    return v;
}

struct Split {
    Tensor part_pointer;
    int64_t num_parts;
};

Split split(const Tensor& node_deg, int64_t num_edges, int part_size)
{
    CHECK_I32(node_deg);
    TORCH_CHECK(part_size >= 1, "back_part_size must be >= 1");
    TORCH_CHECK(num_edges >= 0, "num_edges must be >= 0");
    Split s{torch::empty({num_edges + 1}, node_deg.options()), 0};
    const size_t bytes = eppgcn_split_workspace_bytes(node_deg.numel());
    auto ws = workspace(bytes, node_deg);
    check(eppgcn_split_back_part(i32(node_deg), static_cast<int>(node_deg.numel()), part_size,
                                 s.part_pointer.data_ptr<int32_t>(), num_edges + 1, ws.data_ptr(), bytes, nullptr,
                                 &s.num_parts, nullptr, stream_of(node_deg)),
          "split_back_part");
    return s;
}

std::vector<Tensor> compact_back_edge(Tensor edge_mask, Tensor column_index)
{
    auto c = compact(edge_mask, column_index);
    auto info = torch::zeros({1}, torch::kFloat64);
    info[0] = static_cast<double>(c.valid_len);
    return {c.id, c.edge_list, info};
}

// Addition: mask_forward and compact_back_edge of one layer in one pass, same arguments as
// mask_forward minus the edge mask and the launch hints; returns what compact_back_edge returns.
std::vector<Tensor> mark_compact(Tensor id, Tensor partPointer, Tensor edgeList, Tensor src_mask, Tensor ngh_mask,
                                 Tensor node_degs, int num_layers, int layer)
{
    CHECK_I32(id); CHECK_I32(partPointer); CHECK_I32(edgeList); CHECK_MASK(src_mask); CHECK_MASK(ngh_mask);
    CHECK_I32(node_degs);
    const bool is_last = layer == num_layers;
    TORCH_CHECK(partPointer.numel() >= id.numel() + 1, "partPointer needs num_parts + 1 entries");
    TORCH_CHECK(src_mask.numel() == node_degs.numel(), "src_mask and node_degs must have one entry per vertex");
    CHECK_COUNTS(edgeList, node_degs.numel());
    TORCH_CHECK(is_last || ngh_mask.numel() == node_degs.numel(), "ngh_mask must have one entry per vertex");
    const int64_t length = edgeList.numel();
    auto out_id = torch::empty({length}, edgeList.options());
    auto out_edge = torch::empty({length}, edgeList.options());
    const size_t nbytes = eppgcn_mark_compact_workspace_bytes(length);
    auto ws = torch::empty({static_cast<int64_t>((nbytes + 7) / 8)}, edgeList.options().dtype(torch::kInt64));
    int64_t valid_len = 0;
    check(eppgcn_mark_compact(i32(id), i32(partPointer), i32(edgeList), static_cast<const uint8_t*>(src_mask.data_ptr()),
                              ngh_mask.numel() ? static_cast<uint8_t*>(ngh_mask.data_ptr()) : nullptr,
                              node_degs.data_ptr<int32_t>(), length ? out_id.data_ptr<int32_t>() : nullptr,
                              length ? out_edge.data_ptr<int32_t>() : nullptr, static_cast<int>(id.numel()), length,
                              is_last ? 1 : 0, ws.data_ptr(), nbytes, nullptr, &valid_len, stream_of(id)),
          "mark_compact");
    auto info = torch::zeros({1}, torch::kFloat64);
    info[0] = static_cast<double>(valid_len);
    return {out_id, out_edge, info};
}

int get_map_back_part_size(Tensor node_deg, int valid_len)
{
    int fell_back = 0;
    const int ps = eppgcn_auto_back_part_size(valid_nodes(node_deg), valid_len, &fell_back);
    if (fell_back)
        TORCH_WARN_ONCE("get_map_back_part_size: the fitted regression gives a group size below 1 for this path (it "
                        "was fitted on small graphs); using the rule fitted for the wave64 kernels instead: ", ps);
    return ps;
}

// The group-size rule re-fitted for the wave64 kernels (no counterpart in the reference's module).
int get_wave64_back_part_size(Tensor node_deg, int valid_len)
{
    return eppgcn_wave64_back_part_size(valid_nodes(node_deg), valid_len);
}

std::vector<Tensor> split_back_part(Tensor node_deg, int num_edges, int back_part_size)
{
    auto s = split(node_deg, num_edges, back_part_size);
    auto info = torch::zeros({1}, torch::kInt32);
    info[0] = static_cast<int>(s.num_parts);
    return {s.part_pointer, info};
}

// Legacy all-in-one (EPPGCN.cpp:229-280): compaction, threshold rule when back_part_size == 0, split.
std::vector<Tensor> build_back_part(Tensor edge_mask, Tensor column_index, Tensor node_deg, int back_part_size, int dim)
{
    (void)dim;
    auto c = compact(edge_mask, column_index);
    if (back_part_size == 0) {
        back_part_size = eppgcn_threshold_back_part_size(valid_nodes(node_deg), c.valid_len);
        TORCH_CHECK(back_part_size > 0, "build_back_part: the threshold rule has no group size for an average kept "
                                        "degree >= 512; pass back_part_size explicitly");
    }
    auto s = split(node_deg, edge_mask.numel(), back_part_size);
    auto info = torch::zeros({2}, torch::kFloat64);
    info[0] = static_cast<double>(back_part_size);
    info[1] = static_cast<double>(s.num_parts);
    return {c.id, c.edge_list, s.part_pointer, info};
}

Tensor get_ginfo(Tensor node_deg, int valid_len)
{
    // the reference reads node_deg on the host (EPPGCN.cpp:351-386) and its caller passes a CPU tensor
    TORCH_CHECK(node_deg.scalar_type() == torch::kInt32, "node_deg must be int32");
    if (!node_deg.is_cuda()) node_deg = node_deg.to(torch::kCUDA);
    node_deg = node_deg.contiguous();
    CHECK_I32(node_deg);
    auto hist = torch::empty({10}, node_deg.options());
    auto re = torch::zeros({10}, torch::kFloat32);
    check(eppgcn_get_ginfo(i32(node_deg), node_deg.numel(), valid_len, hist.data_ptr<int32_t>(), re.data_ptr<float>(),
                           stream_of(node_deg)),
          "get_ginfo");
    return re;
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    namespace py = pybind11;
    // the trailing keyword arguments are additions: relu_input applies max(x, 0) to the layer input
    // inside the product (and masks dX accordingly); need_dx=False skips dX (an empty tensor is returned)
    m.def("forward", &forward, "neighbour-group forward: X*W + aggregation (HIP)", py::arg("input"), py::arg("weight"),
          py::arg("row_pointers"), py::arg("column_index"), py::arg("degrees"), py::arg("part_pointers"),
          py::arg("part2Node"), py::arg("partSize"), py::arg("dimWorker"), py::arg("warpPerBlock"),
          py::arg("relu_input") = false);
    m.def("backward", &backward, "unpruned backward: aggregation + dX, dW (HIP)", py::arg("d_output"), py::arg("X"),
          py::arg("W"), py::arg("row_pointers"), py::arg("column_index"), py::arg("degrees"), py::arg("part_pointers"),
          py::arg("part2Node"), py::arg("partSize"), py::arg("dimWorker"), py::arg("warpPerBlock"),
          py::arg("need_dx") = true, py::arg("relu_input") = false);
    m.def("mask_forward", &mask_forward, "mark the backward execution path of one layer (HIP)");
    m.def("ours_backward", &ours_backward, "pruned backward over the compacted path: aggregation + dX, dW (HIP)",
          py::arg("d_output"), py::arg("X"), py::arg("W"), py::arg("id"), py::arg("partPointer"), py::arg("edgeList"),
          py::arg("degrees"), py::arg("partSize"), py::arg("numParts"), py::arg("layer"), py::arg("blockx"),
          py::arg("blocky"), py::arg("need_dx") = true, py::arg("relu_input") = false);
    m.def("set_dense_policy", [](int policy) { g_dense_policy = policy; },
          "dense products: 0 = library kernels where the shapes fit (default), -1 = always torch::mm");
    m.def("set_masked_update", [](bool on) { g_masked_update = on ? 1 : 0; },
          "pruned backward: true (default) = the dense products take the bitmap of the rows the aggregation wrote and the "
          "other rows are neither cleared nor read; false = clear and read every row");
    m.def("print_time", &eppgcn_print_time, "print accumulated kernel times");
    m.def("clear_time", &eppgcn_clear_time, "reset accumulated kernel times");
    m.def("set_timing", [](bool on) { eppgcn_set_timing(on ? 1 : 0); }, "enable per-call kernel timing");
    m.def("aggregation_status",
          []() { check(eppgcn_aggregation_status(static_cast<void*>(c10::hip::getCurrentHIPStream().stream())), "aggregation_status"); },
          "synchronise and raise if a planned aggregation call found its plan's memory replaced (see eppgcn_hip.h)");
    m.def("get_time_ms", &eppgcn_get_time_ms, "accumulated kernel time in ms");
    m.def("clear_plans", []() { drop_all_plans(); g_path_choices.clear(); }, "drop the cached execution plans");
    m.def("set_plan_policy", [](int policy) { g_plan_policy = policy; drop_all_plans(); g_path_choices.clear(); },
          "execution plans: 0 = where the feature table outgrows the caches (default), 1 = always, -1 = never");
    m.def("cached_plans", []() { return static_cast<int>(g_plans.size()); }, "number of execution plans held");

    m.def("build_part", &build_part, "forward neighbour groups (HIP)");
    m.def("build_back_part", &build_back_part, "compaction + group split in one call (HIP)");
    m.def("compact_back_edge", &compact_back_edge, "compact the kept edges of one layer (HIP)");
    m.def("mark_compact", &mark_compact, "marking + compaction of one layer in one pass (HIP)");
    m.def("get_map_back_part_size", &get_map_back_part_size, "backward group size from the fitted regression");
    m.def("get_wave64_back_part_size", &get_wave64_back_part_size, "backward group size re-fitted for wave64 kernels");
    m.def("split_back_part", &split_back_part, "split kept edges into backward groups (HIP)");
    m.def("get_ginfo", &get_ginfo, "degree-distribution features of the kept path");
}
