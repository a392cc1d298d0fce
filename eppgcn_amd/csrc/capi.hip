// extern "C" entry points of libeppgcn_hip.so: argument checks, timers and the
// host halves (count read-back, heuristics) of the aggregation path.
#include "../../include/eppgcn_hip_tuning.h"

#include <atomic>
#include <cmath>
#include <cstdio>
#include <cstring>

#include "common.hpp"

namespace eppgcn {

// ---- implemented in aggregate.hip / prepare.hip
int aggregate_forward_groups(float*, const float*, const int*, const float*, const int*, const int*, const void*, int,
                             int, int, int, float*, size_t, hipStream_t, double*, double*);
int aggregate_compacted_groups(float*, const float*, const int*, const int*, const int*, const float*, const void*,
                               int, int, int, int, float*, size_t, const uint32_t*, hipStream_t, double*, double*,
                               const uint32_t** written = nullptr, long long* num_written = nullptr);
size_t plan_workspace_bytes(long long, long long);
int read_plan_status(const void*, long long, long long, long long, long long*, hipStream_t);
void set_stream_mode(int);
int last_call_used_stream();
int schedule_shift(int);
void set_schedule_shift(int);
void set_plan_keep_rows(int);
void set_plan_length_classes(int);
int launch_build_plan(const int*, const int*, const int*, const int*, int, long long, int, int, int, void*, size_t,
                      void*, size_t, hipStream_t);
void set_agg_force_team(int);
void set_agg_force_rounds(int);
size_t feature_workspace_floats(long long, int);
int workspace_pitch(int);
int launch_dense_rows(float*, int, int, const float*, int, const float*, long long, long long, const float*,
                      const float*, int, int, long long, int, int, hipStream_t, unsigned, const uint32_t* rows = nullptr);
size_t update_workspace_bytes(long long, int, int);
int launch_dense_weight(float*, const float*, int, const float*, int, int, long long, int, int, void*, hipStream_t,
                        const uint32_t* rows = nullptr);
bool dense_backward_fused_covers(int, int, const float*, const float*);
int launch_dense_backward(float*, float*, const float*, const float*, const float*, int, long long, int, int, void*,
                          hipStream_t, const uint32_t* rows = nullptr);
size_t compact_workspace_bytes(long long);
size_t split_workspace_bytes(long long);
int launch_mask_forward(const int*, const int*, const int*, const uint8_t*, uint8_t*, int*, int*, int, long long, int,
                        hipStream_t);
int launch_compact_mask(const int*, int*, const int*, int*, long long, void*, hipStream_t);
long long static_compact_max_length();
int launch_compact_mask_static(const int*, int*, const int*, int*, long long, void**, hipStream_t);
int static_compact_workspace(void**);
int read_aggregation_status(hipStream_t);
size_t mark_compact_workspace_bytes(long long);
int launch_mark_compact(const int*, const int*, const int*, const uint8_t*, uint8_t*, int*, int*, int*, int, long long,
                        int, void*, hipStream_t);
int launch_split(bool, const int*, int, int, int*, int*, long long, bool, void*, hipStream_t);
int launch_count_nonzero(const int*, long long, int*, hipStream_t);
int launch_ginfo_hist(const int*, long long, int*, hipStream_t);
int launch_mark_listed_rows(const int*, long long, long long, uint32_t*, int*, hipStream_t);
// ---- errors
static thread_local std::string g_last_error;
void set_error(const std::string& msg) { g_last_error = msg; }
int hip_fail(hipError_t e, const char* what)
{
    g_last_error = std::string(what) + ": " + hipGetErrorString(e);
    return kErrHip;
}

// ---- timers (milliseconds)
constexpr int kMaxTimedLayers = 16;
static std::atomic<bool> g_timing{false};
static double g_for_agg_ms = 0.0, g_back_agg_ms = 0.0, g_mask_ms = 0.0;
static double g_layer_back_ms[kMaxTimedLayers] = {0};

static double g_phase_ms[2] = {0.0, 0.0};       // output clears, pre-scaling passes of the aggregation calls

bool timing_enabled() { return g_timing.load(); }
double* phase_sink(int which) { return &g_phase_ms[which & 1]; }

static int read_state(void* workspace, hipStream_t stream, ScanState* host)
{
    EPPGCN_HIP(hipMemcpyAsync(host, workspace, sizeof(ScanState), hipMemcpyDeviceToHost, stream));
    EPPGCN_HIP(hipStreamSynchronize(stream));
    if (host->error) {
        set_error("look-back scan stalled: a tile waited past its spin limit; results are invalid");
        return kErrScanStalled;
    }
    return kOk;
}

static bool aligned(const void* p, size_t a) { return reinterpret_cast<uintptr_t>(p) % a == 0; }

}  // namespace eppgcn

using namespace eppgcn;

extern "C" {

const char* eppgcn_last_error(void) { return g_last_error.c_str(); }
int eppgcn_abi_version(void) { return 16; }

int eppgcn_spmm_forward(float* out, const float* in, const int32_t* row_pointers, const int32_t* column_index,
                        const float* degrees, const int32_t* part_pointers, const int32_t* part2node, int num_nodes,
                        int dim, int num_parts, int part_size, int dim_worker, int warp_per_block, float* workspace,
                        size_t workspace_floats, const void* plan, void* stream)
{
    (void)row_pointers;
    EPPGCN_REQUIRE(num_nodes >= 0 && dim > 0 && num_parts >= 0, "num_nodes >= 0, dim > 0, num_parts >= 0 required");
    EPPGCN_REQUIRE(part_size > 0 && dim_worker > 0 && warp_per_block > 0, "launch hints must be positive");
    if (num_nodes == 0) return kOk;
    EPPGCN_REQUIRE(out && (in || workspace) && degrees, "null feature or scale pointer");
    EPPGCN_REQUIRE(num_parts == 0 || (column_index && part_pointers && part2node), "null index pointer");
    EPPGCN_REQUIRE(aligned(out, 4) && aligned(in, 4), "feature pointers must be 4-byte aligned");
    EPPGCN_REQUIRE(!plan || aligned(plan, 256), "plan must be 256-byte aligned");
    EPPGCN_REQUIRE(!workspace || (aligned(workspace, 16) && workspace != out),
                   "workspace must be 16-byte aligned and distinct from the output");
    EPPGCN_REQUIRE(!workspace || workspace == in || workspace_floats >= feature_workspace_floats(num_nodes, dim),
                   "workspace smaller than eppgcn_feature_workspace_floats(num_nodes, dim)");
    return aggregate_forward_groups(out, in, column_index, degrees, part_pointers, part2node, plan, num_nodes, dim,
                                    num_parts, part_size, workspace, workspace_floats, static_cast<hipStream_t>(stream),
                                    &g_for_agg_ms, nullptr);
}

int eppgcn_spmm_backward(float* d_input, const float* d_output, const int32_t* row_pointers,
                         const int32_t* column_index, const float* degrees, const int32_t* part_pointers,
                         const int32_t* part2node, int num_nodes, int dim, int num_parts, int part_size, int dim_worker,
                         int warp_per_block, float* workspace, size_t workspace_floats, const void* plan, void* stream)
{
    (void)row_pointers;
    EPPGCN_REQUIRE(num_nodes >= 0 && dim > 0 && num_parts >= 0, "num_nodes >= 0, dim > 0, num_parts >= 0 required");
    EPPGCN_REQUIRE(part_size > 0 && dim_worker > 0 && warp_per_block > 0, "launch hints must be positive");
    if (num_nodes == 0) return kOk;
    EPPGCN_REQUIRE(d_input && (d_output || workspace) && degrees, "null feature or scale pointer");
    EPPGCN_REQUIRE(num_parts == 0 || (column_index && part_pointers && part2node), "null index pointer");
    EPPGCN_REQUIRE(aligned(d_input, 4) && aligned(d_output, 4), "feature pointers must be 4-byte aligned");
    EPPGCN_REQUIRE(!plan || aligned(plan, 256), "plan must be 256-byte aligned");
    EPPGCN_REQUIRE(!workspace || (aligned(workspace, 16) && workspace != d_input),
                   "workspace must be 16-byte aligned and distinct from the output");
    EPPGCN_REQUIRE(!workspace || workspace == d_output || workspace_floats >= feature_workspace_floats(num_nodes, dim),
                   "workspace smaller than eppgcn_feature_workspace_floats(num_nodes, dim)");
    return aggregate_forward_groups(d_input, d_output, column_index, degrees, part_pointers, part2node, plan,
                                    num_nodes, dim, num_parts, part_size, workspace, workspace_floats,
                                    static_cast<hipStream_t>(stream), &g_back_agg_ms, nullptr);
}

// shared by the two pruned-backward entry points; written == nullptr: the plain call (every row of d_input defined)
static int ours_backward_call(float* d_input, const float* d_output, const int32_t* ids, const int32_t* part_pointer,
                              const int32_t* edge_list, const float* degrees, int num_nodes, int dim, int num_parts,
                              int part_size, int layer, int blockx, int blocky, float* workspace,
                              size_t workspace_floats, const void* plan, const uint32_t* gathered_rows,
                              const uint32_t** written, long long* num_written, void* stream)
{
    // part_size only sizes the work per wave (the reference's kernel ignores it, EPPGCN_kernel.cu:636)
    EPPGCN_REQUIRE(num_nodes >= 0 && dim > 0 && num_parts >= 0, "num_nodes >= 0, dim > 0, num_parts >= 0 required");
    EPPGCN_REQUIRE(blockx > 0 && blocky > 0, "launch hints must be positive");
    EPPGCN_REQUIRE(layer >= 1, "layer is 1-based");
    if (num_nodes == 0) return kOk;
    EPPGCN_REQUIRE(d_input && (d_output || workspace) && degrees, "null feature or scale pointer");
    EPPGCN_REQUIRE(num_parts == 0 || (ids && part_pointer && edge_list), "null index pointer");
    EPPGCN_REQUIRE(aligned(d_input, 4) && aligned(d_output, 4), "feature pointers must be 4-byte aligned");
    EPPGCN_REQUIRE(!plan || aligned(plan, 256), "plan must be 256-byte aligned");
    EPPGCN_REQUIRE(!workspace || (aligned(workspace, 16) && workspace != d_input),
                   "workspace must be 16-byte aligned and distinct from the output");
    EPPGCN_REQUIRE(!workspace || workspace == d_output || workspace_floats >= feature_workspace_floats(num_nodes, dim),
                   "workspace smaller than eppgcn_feature_workspace_floats(num_nodes, dim)");
    return aggregate_compacted_groups(d_input, d_output, ids, part_pointer, edge_list, degrees, plan, num_nodes,
                                      dim, num_parts, part_size > 0 ? part_size : 1, workspace, workspace_floats, gathered_rows,
                                      static_cast<hipStream_t>(stream), &g_back_agg_ms,
                                      layer <= kMaxTimedLayers ? &g_layer_back_ms[layer - 1] : nullptr, written, num_written);
}

int eppgcn_ours_backward(float* d_input, const float* d_output, const int32_t* ids, const int32_t* part_pointer,
                         const int32_t* edge_list, const float* degrees, int num_nodes, int dim, int num_parts,
                         int part_size, int layer, int blockx, int blocky, float* workspace,
                         size_t workspace_floats, const void* plan, const uint32_t* gathered_rows, void* stream)
{
    return ours_backward_call(d_input, d_output, ids, part_pointer, edge_list, degrees, num_nodes, dim, num_parts, part_size,
                              layer, blockx, blocky, workspace, workspace_floats, plan, gathered_rows, nullptr, nullptr, stream);
}

int eppgcn_ours_backward_rows(float* d_input, const float* d_output, const int32_t* ids, const int32_t* part_pointer,
                              const int32_t* edge_list, const float* degrees, int num_nodes, int dim, int num_parts,
                              int part_size, int layer, int blockx, int blocky, float* workspace,
                              size_t workspace_floats, const void* plan, const uint32_t* gathered_rows,
                              const uint32_t** written_rows, int64_t* num_written, void* stream)
{
    EPPGCN_REQUIRE(written_rows, "written_rows must not be NULL (eppgcn_ours_backward is the call without it)");
    *written_rows = nullptr;
    if (num_written) *num_written = num_nodes > 0 ? num_nodes : 0;
    long long count = num_nodes;
    const int rc = ours_backward_call(d_input, d_output, ids, part_pointer, edge_list, degrees, num_nodes, dim, num_parts,
                                      part_size, layer, blockx, blocky, workspace, workspace_floats, plan, gathered_rows,
                                      written_rows, &count, stream);
    if (rc == kOk && num_written && *written_rows) *num_written = count;
    return rc;
}

int eppgcn_mask_forward(const int32_t* part2node, const int32_t* part_pointers, const int32_t* column_index,
                        const uint8_t* src_mask, uint8_t* ngh_mask, int32_t* back_edge_mask, int32_t* node_degs,
                        int num_parts, int64_t num_edges, int is_last_layer, int blockx, int blocky, void* stream)
{
    EPPGCN_REQUIRE(num_parts >= 0 && num_edges >= 0, "negative size");
    EPPGCN_REQUIRE(blockx > 0 && blocky > 0, "launch hints must be positive");
    if (num_parts == 0) return kOk;
    EPPGCN_REQUIRE(part2node && part_pointers && column_index && src_mask && back_edge_mask && node_degs,
                   "null pointer");
    EPPGCN_REQUIRE(is_last_layer || ngh_mask, "ngh_mask may only be NULL on the last layer");
    KernelTimer t(static_cast<hipStream_t>(stream), &g_mask_ms);
    return launch_mask_forward(part2node, part_pointers, column_index, src_mask, ngh_mask, back_edge_mask, node_degs,
                               num_parts, num_edges, is_last_layer ? 1 : 0, static_cast<hipStream_t>(stream));
}

size_t eppgcn_feature_workspace_floats(int64_t num_nodes, int dim)
{
    return (num_nodes <= 0 || dim <= 0) ? 0 : feature_workspace_floats(num_nodes, dim);
}
int eppgcn_plan_recommended(int64_t num_nodes, int dim)
{
    if (num_nodes <= 0 || dim <= 0) return 0;
    return static_cast<double>(feature_workspace_floats(num_nodes, dim)) * 4.0 >= 4.0 * (1 << 20) ? 1 : 0;
}
size_t eppgcn_plan_bytes(int64_t num_parts, int64_t num_slots, int64_t num_nodes)
{
    return plan_bytes(num_parts, num_slots, num_nodes);
}
size_t eppgcn_plan_workspace_bytes(int64_t num_parts, int64_t num_slots)
{
    return plan_workspace_bytes(num_parts, num_slots);
}

int eppgcn_build_plan(const int32_t* part_pointers, const int32_t* column_index, const int32_t* part2node,
                      const int32_t* ids, int num_parts, int64_t num_slots, int num_nodes, int dim, int block_shift,
                      void* plan, size_t plan_size, void* workspace, size_t workspace_bytes, void* stream)
{
    EPPGCN_REQUIRE(num_parts >= 0 && num_slots >= 0 && num_nodes >= 0 && dim > 0, "negative size");
    EPPGCN_REQUIRE(block_shift >= 0 && block_shift <= 31, "block_shift must be 0 (automatic) or 1..31");
    if (num_parts == 0) return kOk;
    EPPGCN_REQUIRE(part_pointers && column_index && plan, "null pointer");
    EPPGCN_REQUIRE((part2node != nullptr) != (ids != nullptr), "give exactly one of part2node (forward) and ids (backward)");
    EPPGCN_REQUIRE(aligned(plan, 256) && workspace && aligned(workspace, 256), "plan and workspace must be 256-byte aligned");
    return launch_build_plan(part_pointers, column_index, part2node, ids, num_parts, num_slots, num_nodes,
                             block_shift > 0 ? block_shift : schedule_shift(dim), dim, plan, plan_size, workspace,
                             workspace_bytes, static_cast<hipStream_t>(stream));
}

size_t eppgcn_compact_workspace_bytes(int64_t length) { return compact_workspace_bytes(length < 0 ? 0 : length); }
size_t eppgcn_split_workspace_bytes(int64_t num_nodes) { return split_workspace_bytes(num_nodes < 0 ? 0 : num_nodes); }

int eppgcn_compact_back_edge(const int32_t* edge_mask, const int32_t* column_index, int32_t* out_id, int32_t* out_edge,
                             int64_t length, void* workspace, size_t workspace_bytes, int32_t* d_valid_len,
                             int64_t* h_valid_len, void* stream)
{
    EPPGCN_REQUIRE(length >= 0 && length < (1ll << 31), "length must fit int32");
    EPPGCN_REQUIRE(workspace && aligned(workspace, 8), "workspace must be 8-byte aligned");
    EPPGCN_REQUIRE(workspace_bytes >= compact_workspace_bytes(length), "workspace too small");
    EPPGCN_REQUIRE(length == 0 || (edge_mask && column_index && out_id && out_edge), "null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (int rc = launch_compact_mask(edge_mask, out_id, column_index, out_edge, length, workspace, s)) return rc;
    ScanState* st = static_cast<ScanState*>(workspace);
    if (d_valid_len)
        EPPGCN_HIP(hipMemcpyAsync(d_valid_len, st->counts, sizeof(int), hipMemcpyDeviceToDevice, s));
    if (h_valid_len) {
        ScanState host;
        if (int rc = read_state(workspace, s, &host)) return rc;
        *h_valid_len = host.counts[0];
    }
    return kOk;
}

int64_t eppgcn_compact_back_edge_static_max_length(void) { return static_compact_max_length(); }

int eppgcn_compact_back_edge_static(const int32_t* edge_mask, const int32_t* column_index, int32_t* out_id,
                                    int32_t* out_edge, int64_t length, int32_t* d_valid_len, int64_t* h_valid_len,
                                    void* stream)
{
    EPPGCN_REQUIRE(length >= 0, "length must not be negative");
    if (length > static_compact_max_length()) {
        set_error("eppgcn_compact_back_edge_static: length " + std::to_string(length) + " exceeds the static scratch (" +
                  std::to_string(static_compact_max_length()) +
                  " slots at most); use eppgcn_compact_back_edge with a caller workspace");
        return kErrCapacity;
    }
    EPPGCN_REQUIRE(length == 0 || (edge_mask && column_index && out_id && out_edge), "null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    void* workspace = nullptr;
    if (int rc = launch_compact_mask_static(edge_mask, out_id, column_index, out_edge, length, &workspace, s)) return rc;
    ScanState* st = static_cast<ScanState*>(workspace);
    if (d_valid_len)
        EPPGCN_HIP(hipMemcpyAsync(d_valid_len, st->counts, sizeof(int), hipMemcpyDeviceToDevice, s));
    if (h_valid_len) {
        ScanState host;
        if (int rc = read_state(workspace, s, &host)) return rc;
        *h_valid_len = host.counts[0];
    }
    return kOk;
}

size_t eppgcn_mark_compact_workspace_bytes(int64_t num_edges) { return mark_compact_workspace_bytes(num_edges); }

int eppgcn_mark_compact(const int32_t* part2node, const int32_t* part_pointers, const int32_t* column_index,
                        const uint8_t* src_mask, uint8_t* ngh_mask, int32_t* node_degs, int32_t* out_id,
                        int32_t* out_edge, int num_parts, int64_t num_edges, int is_last, void* workspace,
                        size_t workspace_bytes, int32_t* d_valid_len, int64_t* h_valid_len, void* stream)
{
    EPPGCN_REQUIRE(num_parts >= 0 && num_edges >= 0 && num_edges < (1ll << 31), "num_parts >= 0 and 0 <= num_edges < 2^31 required");
    EPPGCN_REQUIRE(workspace && aligned(workspace, 8), "workspace must be 8-byte aligned");
    EPPGCN_REQUIRE(workspace_bytes >= mark_compact_workspace_bytes(num_edges), "workspace too small");
    EPPGCN_REQUIRE(num_edges == 0 || (out_id && out_edge), "null output pointer");
    EPPGCN_REQUIRE(num_parts == 0 || (part2node && part_pointers && column_index && src_mask && node_degs),
                   "null pointer");
    EPPGCN_REQUIRE(is_last || num_parts == 0 || ngh_mask, "ngh_mask is required unless this is the last layer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    {
        KernelTimer timer(s, &g_mask_ms);
        if (int rc = launch_mark_compact(part2node, part_pointers, column_index, src_mask, ngh_mask, node_degs, out_id,
                                         out_edge, num_parts, num_edges, is_last ? 1 : 0, workspace, s))
            return rc;
    }
    ScanState* st = static_cast<ScanState*>(workspace);
    if (d_valid_len)
        EPPGCN_HIP(hipMemcpyAsync(d_valid_len, st->counts, sizeof(int), hipMemcpyDeviceToDevice, s));
    if (h_valid_len) {
        ScanState host;
        if (int rc = read_state(workspace, s, &host)) return rc;
        *h_valid_len = host.counts[0];
    }
    return kOk;
}

int eppgcn_mark_gathered_rows(const int32_t* edge_list, int64_t valid_len, int num_nodes, uint32_t* bitmap,
                              int32_t* d_count, int64_t* h_count, void* stream)
{
    EPPGCN_REQUIRE(valid_len >= 0 && valid_len < (1ll << 31) && num_nodes >= 0, "lengths must be non-negative int32");
    EPPGCN_REQUIRE(d_count && (num_nodes == 0 || bitmap) && (valid_len == 0 || edge_list), "null pointer");
    EPPGCN_REQUIRE(aligned(bitmap, 4) && aligned(d_count, 4), "bitmap and counter must be 4-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (int rc = launch_mark_listed_rows(edge_list, valid_len, num_nodes, bitmap, d_count, s)) return rc;
    if (h_count) {
        int v = 0;
        EPPGCN_HIP(hipMemcpyAsync(&v, d_count, sizeof(int), hipMemcpyDeviceToHost, s));
        EPPGCN_HIP(hipStreamSynchronize(s));
        *h_count = v;
    }
    return kOk;
}

int eppgcn_count_nonzero(const int32_t* node_deg, int64_t length, int32_t* d_count, int64_t* h_count, void* stream)
{
    EPPGCN_REQUIRE(length >= 0 && length < (1ll << 31), "length must fit int32");
    EPPGCN_REQUIRE(d_count && (length == 0 || node_deg), "null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (int rc = launch_count_nonzero(node_deg, length, d_count, s)) return rc;
    if (h_count) {
        int v = 0;
        EPPGCN_HIP(hipMemcpyAsync(&v, d_count, sizeof(int), hipMemcpyDeviceToHost, s));
        EPPGCN_HIP(hipStreamSynchronize(s));
        *h_count = v;
    }
    return kOk;
}

int eppgcn_map_back_part_size(int64_t valid_node, int64_t valid_len, int* clamped)
{
    if (clamped) *clamped = 0;
    if (valid_node <= 0) {
        if (clamped) *clamped = 1;
        return 1;
    }
    const double valid_degree = 1.0 * static_cast<double>(valid_len) / static_cast<double>(valid_node);
    const double beta0 = 0.65538, beta1 = 1.67431e-5, beta2 = -2.24342e-6, beta3 = 0.63641;
    const double raw = std::round(beta0 + beta1 * static_cast<double>(valid_node) +
                                  beta2 * static_cast<double>(valid_len) + beta3 * valid_degree);
    if (raw < 1.0) {
        if (clamped) *clamped = 1;
        return 1;
    }
    return static_cast<int>(raw);
}

int eppgcn_threshold_back_part_size(int64_t valid_node, int64_t valid_len)
{
    if (valid_node <= 0) return 4;
    const int64_t valid_degree = valid_len / valid_node;
    if (valid_degree < 4) return 4;
    if (valid_degree < 16) return 8;
    if (valid_degree < 64) return 16;
    if (valid_degree < 256) return 32;
    if (valid_degree < 512) return 64;
    return 0;
}

int eppgcn_wave64_back_part_size(int64_t valid_node, int64_t valid_len)
{
    // measured on R-MAT scale 20 and 22, mask ratios 0.01-0.5, widths 16-256: 16 is best or within 2 % of the
    // best up to an average kept degree of about 20, 32 above (first-layer paths with 30 kept edges per row:
    // 8 / 16 / 32 / 64 / 128 -> 1.97 / 1.42 / 1.21 / 1.30 / 1.63 ms)
    if (valid_node <= 0) return 16;
    return valid_len / valid_node < 24 ? 16 : 32;
}

int eppgcn_auto_back_part_size(int64_t valid_node, int64_t valid_len, int* fell_back)
{
    int clamped = 0;
    const int fitted = eppgcn_map_back_part_size(valid_node, valid_len, &clamped);
    if (fell_back) *fell_back = clamped;
    return clamped ? eppgcn_wave64_back_part_size(valid_node, valid_len) : fitted;
}

int eppgcn_scan_status(const void* workspace, void* stream)
{
    if (!workspace) {       // the static scratch of eppgcn_compact_back_edge_static on the current device
        void* ws = nullptr;
        if (int rc = static_compact_workspace(&ws)) return rc;
        workspace = ws;
    }
    EPPGCN_REQUIRE(aligned(workspace, 8), "workspace must be 8-byte aligned");
    ScanState host;
    if (int rc = read_state(const_cast<void*>(workspace), static_cast<hipStream_t>(stream), &host)) return rc;
    if (host.overflow) {
        set_error("group pointers did not fit the given capacity (need " + std::to_string(host.counts[0] + 1) +
                  " entries)");
        return kErrCapacity;
    }
    return kOk;
}

int eppgcn_plan_status(const void* plan, int num_parts, int64_t num_slots, int num_nodes, int64_t* partial_rows,
                       void* stream)
{
    EPPGCN_REQUIRE(num_parts >= 0 && num_slots >= 0 && num_nodes >= 0, "negative size");
    if (partial_rows) *partial_rows = 0;
    if (num_parts == 0) return kOk;
    EPPGCN_REQUIRE(plan && aligned(plan, 256), "plan must be 256-byte aligned");
    long long partial = 0;
    const int rc = read_plan_status(plan, num_parts, num_slots, num_nodes, &partial, static_cast<hipStream_t>(stream));
    if (partial_rows) *partial_rows = partial;
    return rc;
}

void eppgcn_plan_release(const void* plan)
{
    if (plan) forget_stream_info(plan);
}

int eppgcn_aggregation_status(void* stream) { return read_aggregation_status(static_cast<hipStream_t>(stream)); }

size_t eppgcn_plan_workspace_floats(const void* plan, int64_t num_nodes, int dim)
{
    size_t rows = static_cast<size_t>(swizzle_padded_rows(num_nodes));
    StreamInfo info;
    if (plan && find_stream_info(plan, &info) && info.header.valid) rows += static_cast<size_t>(info.header.num_partials);
    return rows * static_cast<size_t>(dim > 0 ? workspace_pitch(dim) : 0);
}

void eppgcn_set_stream_mode(int on) { set_stream_mode(on); }
int eppgcn_last_call_used_stream(void) { return last_call_used_stream(); }

static int finish_split(void* workspace, hipStream_t s, int32_t* d_counts, int64_t* h_a, int64_t* h_b)
{
    ScanState* st = static_cast<ScanState*>(workspace);
    if (d_counts) EPPGCN_HIP(hipMemcpyAsync(d_counts, st->counts, 2 * sizeof(int), hipMemcpyDeviceToDevice, s));
    if (h_a || h_b) {
        ScanState host;
        if (int rc = read_state(workspace, s, &host)) return rc;
        if (h_a) *h_a = host.counts[0];
        if (h_b) *h_b = host.counts[1];
        if (host.overflow) {
            set_error("group pointers do not fit the given capacity (need " + std::to_string(host.counts[0] + 1) +
                      " entries)");
            return kErrCapacity;
        }
    }
    return kOk;
}

int eppgcn_split_back_part(const int32_t* node_deg, int num_nodes, int part_size, int32_t* part_pointer,
                           int64_t capacity, void* workspace, size_t workspace_bytes, int32_t* d_counts,
                           int64_t* h_num_parts, int64_t* h_valid_len, void* stream)
{
    EPPGCN_REQUIRE(num_nodes >= 0 && part_size >= 1, "num_nodes >= 0 and part_size >= 1 required");
    EPPGCN_REQUIRE(capacity >= 1 && part_pointer, "part_pointer needs at least one entry");
    EPPGCN_REQUIRE(workspace && aligned(workspace, 8), "workspace must be 8-byte aligned");
    EPPGCN_REQUIRE(workspace_bytes >= split_workspace_bytes(num_nodes), "workspace too small");
    EPPGCN_REQUIRE(num_nodes == 0 || node_deg, "null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (int rc = launch_split(false, node_deg, num_nodes, part_size, part_pointer, nullptr, capacity, true, workspace, s))
        return rc;
    return finish_split(workspace, s, d_counts, h_num_parts, h_valid_len);
}

int eppgcn_build_part(const int32_t* row_pointers, int num_nodes, int part_size, int32_t* part_pointers,
                      int32_t* part2node, int64_t capacity, void* workspace, size_t workspace_bytes, int32_t* d_counts,
                      int64_t* h_num_parts, void* stream)
{
    EPPGCN_REQUIRE(num_nodes >= 0 && part_size >= 1, "num_nodes >= 0 and part_size >= 1 required");
    EPPGCN_REQUIRE(capacity >= 1 && part_pointers && (capacity == 1 || part2node), "output buffers required");
    EPPGCN_REQUIRE(workspace && aligned(workspace, 8), "workspace must be 8-byte aligned");
    EPPGCN_REQUIRE(workspace_bytes >= split_workspace_bytes(num_nodes), "workspace too small");
    EPPGCN_REQUIRE(row_pointers, "null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (int rc = launch_split(true, row_pointers, num_nodes, part_size, part_pointers, part2node, capacity, false,
                              workspace, s))
        return rc;
    return finish_split(workspace, s, d_counts, h_num_parts, nullptr);
}

int eppgcn_get_ginfo(const int32_t* node_deg, int64_t num_nodes, int64_t valid_len, int32_t* d_hist, float* h_out,
                     void* stream)
{
    EPPGCN_REQUIRE(num_nodes >= 0 && num_nodes < (1ll << 31), "num_nodes must fit int32");
    EPPGCN_REQUIRE(d_hist && h_out && (num_nodes == 0 || node_deg), "null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (int rc = launch_ginfo_hist(node_deg, num_nodes, d_hist, s)) return rc;
    int hist[10];
    EPPGCN_HIP(hipMemcpyAsync(hist, d_hist, sizeof(hist), hipMemcpyDeviceToHost, s));
    EPPGCN_HIP(hipStreamSynchronize(s));
    // same expressions as the reference: float counts, double divisions, float32 results
    const int valid_node = hist[0];
    h_out[0] = static_cast<float>(valid_node * 1.0 / 10000);
    h_out[1] = static_cast<float>(valid_len * 1.0 / 10000);
    h_out[2] = static_cast<float>(1.0 * valid_len / valid_node);
    for (int i = 3; i < 10; ++i) h_out[i] = static_cast<float>(static_cast<float>(hist[i]) * 1.0 / valid_node);
    return kOk;
}

void eppgcn_set_timing(int enabled) { g_timing.store(enabled != 0); }

void eppgcn_print_time(void)
{
    // same lines as the reference's print_time (EPPGCN_kernel.cu:96-106), in seconds
    std::printf("for_agg_time: %.6f\n", g_for_agg_ms / 1000);
    std::printf("back_agg_time: %.6f\n", g_back_agg_ms / 1000);
    for (int i = 0; i < kMaxTimedLayers && g_layer_back_ms[i] != 0.0; ++i)
        std::printf("l%d_back_agg_time: %.6f\n", i + 1, g_layer_back_ms[i] / 1000);
    std::printf("mask_time: %.6f\n", g_mask_ms / 1000);
    std::fflush(stdout);
}

void eppgcn_clear_time(void)
{
    // the marking time survives a clear, as in the reference (EPPGCN_kernel.cu:108-116): marking
    // runs once during warm-up and is still reported after the timed epochs
    g_for_agg_ms = 0.0;
    g_back_agg_ms = 0.0;
    for (double& v : g_layer_back_ms) v = 0.0;
    g_phase_ms[0] = g_phase_ms[1] = 0.0;
}

double eppgcn_get_time_ms(int which)
{
    if (which == 0) return g_for_agg_ms;
    if (which == 1) return g_back_agg_ms;
    if (which == 2) return g_mask_ms;
    if (which == 3 || which == 4) return g_phase_ms[which - 3];
    if (which > 100 && which <= 100 + kMaxTimedLayers) return g_layer_back_ms[which - 101];
    return -1.0;
}

void eppgcn_set_team_size(int lanes) { set_agg_force_team(lanes); }
void eppgcn_set_rounds(int rounds) { set_agg_force_rounds(rounds); }
void eppgcn_set_wide_index(int on) { set_force_wide_index(on != 0); }
void eppgcn_set_scan_test_mode(unsigned spin_limit, int mute_first_tile) { set_scan_test_mode(spin_limit, mute_first_tile); }
void eppgcn_set_plan_shift(int shift) { set_schedule_shift(shift); }
void eppgcn_set_plan_keep_rows(int groups) { set_plan_keep_rows(groups); }
void eppgcn_set_plan_length_classes(int on) { set_plan_length_classes(on); }

// ---- dense update
int eppgcn_feature_workspace_pitch(int dim) { return dim > 0 ? workspace_pitch(dim) : 0; }

int eppgcn_update_supported(int in_dim, int out_dim)
{
    if (in_dim <= 0 || out_dim <= 0) return 0;
    int mask = 0;
    if (in_dim <= 1024) mask |= 1;       // forward: reduction over in_dim
    if (out_dim <= 1024) mask |= 2;      // backward_input: reduction over out_dim
    if (out_dim <= 64) mask |= 4;        // backward_weight: gradient columns held in one block
    return mask;
}

int eppgcn_update_forward(float* out, int ld_out, const float* x, const float* w, const float* scale,
                          int relu_input, int64_t num_nodes, int in_dim, int out_dim, void* stream)
{
    EPPGCN_REQUIRE(num_nodes >= 0 && in_dim > 0 && out_dim > 0, "num_nodes >= 0, in_dim > 0, out_dim > 0 required");
    EPPGCN_REQUIRE(ld_out >= out_dim, "ld_out must be at least out_dim");
    if (num_nodes == 0) return kOk;
    EPPGCN_REQUIRE(out && x && w, "null matrix pointer");
    EPPGCN_REQUIRE(aligned(out, 4) && aligned(x, 4) && aligned(w, 4), "matrix pointers must be 4-byte aligned");
    EPPGCN_REQUIRE(out != x, "the product cannot be written over its input");
    return launch_dense_rows(out, ld_out, ld_out, x, in_dim, w, out_dim, 1, scale, nullptr, 0, relu_input ? 1 : 0,
                             num_nodes, in_dim, out_dim, static_cast<hipStream_t>(stream), 0u);
}

int eppgcn_update_forward_table(float* table, size_t table_floats, const float* x, const float* w, const float* scale,
                                int relu_input, int64_t num_nodes, int in_dim, int out_dim, void* stream)
{
    EPPGCN_REQUIRE(num_nodes >= 0 && in_dim > 0 && out_dim > 0, "num_nodes >= 0, in_dim > 0, out_dim > 0 required");
    if (num_nodes == 0) return kOk;
    EPPGCN_REQUIRE(table && x && w && scale, "null pointer");
    EPPGCN_REQUIRE(aligned(table, 16) && aligned(x, 4) && aligned(w, 4), "table must be 16-byte, matrices 4-byte aligned");
    EPPGCN_REQUIRE(table != x, "the product cannot be written over its input");
    EPPGCN_REQUIRE(num_nodes < (1ll << 31), "too many rows");
    EPPGCN_REQUIRE(table_floats >= feature_workspace_floats(num_nodes, out_dim),
                   "table smaller than eppgcn_feature_workspace_floats(num_nodes, out_dim)");
    const int pitch = workspace_pitch(out_dim);
    return launch_dense_rows(table, pitch, pitch, x, in_dim, w, out_dim, 1, scale, nullptr, 0, relu_input ? 1 : 0,
                             num_nodes, in_dim, out_dim, static_cast<hipStream_t>(stream), kRowSwizzleMask);
}

int64_t eppgcn_feature_workspace_row(int64_t vertex)
{
    return vertex < 0 ? -1 : static_cast<int64_t>((static_cast<uint64_t>(vertex) & ~0xffffffffull) |
                                                  swizzled_row(static_cast<unsigned>(vertex & 0xffffffffll)));
}

int eppgcn_update_backward_input(float* d_x, const float* g, const float* w, const float* relu_ref,
                                 int64_t num_nodes, int in_dim, int out_dim, void* stream)
{
    EPPGCN_REQUIRE(num_nodes >= 0 && in_dim > 0 && out_dim > 0, "num_nodes >= 0, in_dim > 0, out_dim > 0 required");
    if (num_nodes == 0) return kOk;
    EPPGCN_REQUIRE(d_x && g && w, "null matrix pointer");
    EPPGCN_REQUIRE(aligned(d_x, 4) && aligned(g, 4) && aligned(w, 4) && aligned(relu_ref, 4),
                   "matrix pointers must be 4-byte aligned");
    EPPGCN_REQUIRE(d_x != g, "the product cannot be written over its input");
    // reduction over the out_dim columns of g; operand element (d, k) is w[k, d]
    return launch_dense_rows(d_x, in_dim, in_dim, g, out_dim, w, 1, out_dim, nullptr, relu_ref, in_dim, 0, num_nodes,
                             out_dim, in_dim, static_cast<hipStream_t>(stream), 0u);
}

size_t eppgcn_update_workspace_bytes(int64_t num_nodes, int in_dim, int out_dim)
{
    return update_workspace_bytes(num_nodes, in_dim, out_dim);
}

int eppgcn_update_backward_weight(float* d_w, const float* x, const float* g, int relu_input, int64_t num_nodes,
                                  int in_dim, int out_dim, void* workspace, size_t workspace_bytes, void* stream)
{
    EPPGCN_REQUIRE(num_nodes >= 0 && in_dim > 0 && out_dim > 0, "num_nodes >= 0, in_dim > 0, out_dim > 0 required");
    EPPGCN_REQUIRE(d_w, "null output pointer");
    EPPGCN_REQUIRE(num_nodes == 0 || (x && g), "null matrix pointer");
    EPPGCN_REQUIRE(aligned(d_w, 4) && aligned(x, 4) && aligned(g, 4), "matrix pointers must be 4-byte aligned");
    EPPGCN_REQUIRE(num_nodes == 0 || (workspace && aligned(workspace, 4) &&
                                      workspace_bytes >= update_workspace_bytes(num_nodes, in_dim, out_dim)),
                   "workspace smaller than eppgcn_update_workspace_bytes(num_nodes, in_dim, out_dim)");
    return launch_dense_weight(d_w, x, in_dim, g, out_dim, relu_input ? 1 : 0, num_nodes, in_dim, out_dim, workspace,
                               static_cast<hipStream_t>(stream));
}

int eppgcn_update_backward(float* d_x, float* d_w, const float* x, const float* g, const float* w, int relu_input,
                           int64_t num_nodes, int in_dim, int out_dim, void* workspace, size_t workspace_bytes,
                           void* stream)
{
    EPPGCN_REQUIRE(num_nodes >= 0 && in_dim > 0 && out_dim > 0, "num_nodes >= 0, in_dim > 0, out_dim > 0 required");
    EPPGCN_REQUIRE(d_w, "null output pointer");
    EPPGCN_REQUIRE(num_nodes == 0 || (d_x && x && g && w), "null matrix pointer");
    EPPGCN_REQUIRE(aligned(d_x, 4) && aligned(d_w, 4) && aligned(x, 4) && aligned(g, 4) && aligned(w, 4),
                   "matrix pointers must be 4-byte aligned");
    EPPGCN_REQUIRE(d_x != g && d_x != x, "the input gradient cannot be written over an input");
    EPPGCN_REQUIRE(num_nodes == 0 || (workspace && aligned(workspace, 4) &&
                                      workspace_bytes >= update_workspace_bytes(num_nodes, in_dim, out_dim)),
                   "workspace smaller than eppgcn_update_workspace_bytes(num_nodes, in_dim, out_dim)");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (num_nodes == 0 || dense_backward_fused_covers(in_dim, out_dim, x, g))
        return launch_dense_backward(d_x, d_w, x, g, w, relu_input ? 1 : 0, num_nodes, in_dim, out_dim, workspace, s);
    if (int rc = launch_dense_weight(d_w, x, in_dim, g, out_dim, relu_input ? 1 : 0, num_nodes, in_dim, out_dim,
                                     workspace, s))
        return rc;
    if (num_nodes == 0) return kOk;
    return launch_dense_rows(d_x, in_dim, in_dim, g, out_dim, w, 1, out_dim, nullptr, relu_input ? x : nullptr, in_dim,
                             0, num_nodes, out_dim, in_dim, s, 0u);
}

int eppgcn_update_backward_rows(float* d_x, float* d_w, const float* x, const float* g, const float* w, int relu_input,
                                const uint32_t* rows, int64_t num_nodes, int in_dim, int out_dim, void* workspace,
                                size_t workspace_bytes, void* stream)
{
    EPPGCN_REQUIRE(num_nodes >= 0 && in_dim > 0 && out_dim > 0, "num_nodes >= 0, in_dim > 0, out_dim > 0 required");
    EPPGCN_REQUIRE(d_w, "null output pointer");
    EPPGCN_REQUIRE(num_nodes == 0 || (x && g && (w || !d_x)), "null matrix pointer");
    EPPGCN_REQUIRE(aligned(d_x, 4) && aligned(d_w, 4) && aligned(x, 4) && aligned(g, 4) && aligned(w, 4) && aligned(rows, 4),
                   "matrix pointers and the row bitmap must be 4-byte aligned");
    EPPGCN_REQUIRE(!d_x || (d_x != g && d_x != x), "the input gradient cannot be written over an input");
    EPPGCN_REQUIRE(num_nodes == 0 || (workspace && aligned(workspace, 4) &&
                                      workspace_bytes >= update_workspace_bytes(num_nodes, in_dim, out_dim)),
                   "workspace smaller than eppgcn_update_workspace_bytes(num_nodes, in_dim, out_dim)");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (d_x && (num_nodes == 0 || dense_backward_fused_covers(in_dim, out_dim, x, g)))
        return launch_dense_backward(d_x, d_w, x, g, w, relu_input ? 1 : 0, num_nodes, in_dim, out_dim, workspace, s, rows);
    if (int rc = launch_dense_weight(d_w, x, in_dim, g, out_dim, relu_input ? 1 : 0, num_nodes, in_dim, out_dim,
                                     workspace, s, rows))
        return rc;
    if (num_nodes == 0 || !d_x) return kOk;
    return launch_dense_rows(d_x, in_dim, in_dim, g, out_dim, w, 1, out_dim, nullptr, relu_input ? x : nullptr, in_dim,
                             0, num_nodes, out_dim, in_dim, s, 0u, rows);
}

}  // extern "C"
