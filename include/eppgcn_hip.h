/*
 * C ABI of the MI355X (gfx950) GCN aggregation path: libeppgcn_hip.so.
 *
 * Tensor-free: device pointers, sizes and a HIP stream (passed as void*, a
 * hipStream_t; NULL = the default stream).  These are the entry points a binding
 * of the reference's `GNNAdvisor` extension module needs; each declaration names
 * the reference interface it stands in for (paths relative to the reference
 * checkout, EPPGCN/GCNConv/).  The dense X*W products of the reference's
 * launchers stay with the caller (torch.mm); the library covers aggregation,
 * path marking, compaction and group construction.
 *
 * Conventions
 *   - Every function returns 0 on success or a negative code (EPPGCN_ERR_*);
 *     eppgcn_last_error() then returns a message.  Nothing aborts the process.
 *   - All pointers are DEVICE pointers unless the name starts with h_.
 *     Index data is int32, features fp32 row-major contiguous, masks one byte
 *     per vertex (torch.bool layout).
 *   - Calls are asynchronous on `stream` unless a host result (h_*) is
 *     requested; a function that fills an h_* argument synchronises the stream
 *     first, as the reference's compactors do.  Device-side failures of the
 *     scan-based functions (a stalled look-back, a capacity overflow) are only
 *     reported by such a synchronising call, or by eppgcn_scan_status /
 *     eppgcn_plan_status.
 *   - Scan-based functions need a workspace of at least the number of bytes the
 *     matching *_workspace_bytes() call returns, 8-byte aligned.  The library
 *     itself allocates no device memory.
 *   - The aggregation functions take an optional feature workspace of
 *     eppgcn_feature_workspace_floats(num_nodes, dim) floats, 16-byte aligned
 *     (its size is passed as workspace_floats and checked).  With it the
 *     features are scaled by `degrees` once per call into padded rows (to a
 *     power of two up to 128 bytes, beyond that to whole 32-byte sectors) and
 *     the kernel gathers pre-scaled rows, which removes one random memory
 *     request per edge; with NULL the kernel gathers the
 *     neighbour's scale per edge and needs no scratch.  The workspace may be the
 *     input pointer itself when the caller no longer needs the unscaled input
 *     (it is then overwritten with degrees[r]*in[r,:], unpadded).  A separate
 *     workspace holds the row of vertex r at row eppgcn_feature_workspace_row(r)
 *     (a permutation inside blocks of 4096 rows that spreads the gathers of graphs
 *     with Kronecker-like vertex ids over the memory channels; the size above counts
 *     whole blocks).  With a NULL
 *     input and a workspace, the workspace must already hold the scaled rows
 *     degrees[r]*in[r,:] in that row order at a pitch of eppgcn_feature_workspace_pitch(dim) floats
 *     with zeros in the padding (eppgcn_update_forward_table writes exactly that) and
 *     the scaling pass is skipped.  Results of the modes agree to rounding (a few
 *     ulp per term).
 *   - Limits: vertices and slots (CSR entries, kept edges) are int32 as in the
 *     reference and must stay below 2^31 - 1024 (the kernels step through slot
 *     ranges 1024 at a time before clamping); element offsets into the [N, dim]
 *     matrices are formed in 64 bits, so N * dim may exceed 2^31.  The slot count
 *     of an aggregation call lives on the device (part_pointers[num_parts]), so
 *     that bound is the caller's to keep; the extension module checks it.
 */
#ifndef EPPGCN_HIP_H_
#define EPPGCN_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define EPPGCN_OK 0
#define EPPGCN_ERR_INVALID_ARGUMENT (-1)
#define EPPGCN_ERR_HIP (-2)
#define EPPGCN_ERR_SCAN_STALLED (-3)
#define EPPGCN_ERR_CAPACITY (-4)
#define EPPGCN_ERR_PLAN_MISMATCH (-5)

/* Message of the last failure on the calling thread ("" if none). */
const char* eppgcn_last_error(void);
/* ABI version of this header. */
int eppgcn_abi_version(void);

/* ---------------------------------------------------------------------------
 * Aggregation.
 * ------------------------------------------------------------------------- */

/* Floats a separate feature workspace must hold for [num_nodes, dim] features. */
size_t eppgcn_feature_workspace_floats(int64_t num_nodes, int dim);
/* Row pitch (floats) of that workspace. */
int eppgcn_feature_workspace_pitch(int dim);
/* Row of that workspace which holds the features of `vertex`: vertex ^ ((vertex >> 5) & 4095). */
int64_t eppgcn_feature_workspace_row(int64_t vertex);

/* Execution plan for the aggregation kernels: a copy of the groups (pointers, rows, adjacency
 * flags, column ids) re-ordered by the column block (2^shift vertices, shift chosen from `dim`;
 * pass the widest feature width the plan will be used with) of each group's first slot, original
 * order inside a block.  The aggregation functions accept it as an optional argument (NULL = the
 * groups as given): it changes no result beyond the order of the float additions, only which groups
 * run together, so that the rows gathered at any moment come from one window of the table and are
 * served from L2.  It is used when a feature workspace is given as well.  Build it once per graph and
 * group array:
 *   forward groups : part_pointers + column_index + part2node (ids = NULL)
 *   backward path  : part_pointer + edge_list + ids (part2node = NULL)
 * num_slots = number of slots the groups cover (num_edges, or the kept length).  The plan must
 * be rebuilt when the groups change, and an aggregation call that is given a plan must be given the
 * num_parts and num_nodes the plan was built with (its layout depends on both).  The plan also
 * records, one bit per vertex, the rows that consist of a single non-empty group: the kernel
 * writes those with one plain store, so the output clear of a planned call skips them.
 * block_shift: 0 = column blocks sized for `dim`-wide rows; n > 0 = blocks of 2^n vertices.  31 keeps
 * the groups in one block (original order apart from the length classes): the right choice for a
 * heavily pruned path, whose few gathered rows stay cached anyway.
 *
 * Stream form.  The plan also holds its slots as one stream with the ends of the rows' pieces marked
 * (a piece = consecutive plan entries that continue one another), for a second kernel in which every
 * wave takes the same number of slots, every gather instruction is full whatever the row lengths,
 * and no float atomics are used: pieces that are all of their row and lie inside one wave's 512 slots
 * are stored directly, the others leave partial sums in a scratch area behind the feature table,
 * which a small second kernel adds up row by row in a fixed order.  Results are then the same bits
 * on every run.  An aggregation call takes this path when
 *   - eppgcn_plan_status has been called for the plan (it reads the counts the host needs),
 *   - a separate feature workspace is given (not NULL, not the input itself) that holds at least
 *     eppgcn_plan_workspace_floats(plan, num_nodes, dim) floats (the table plus the partial sums),
 *   - rows are at most 1024 bytes (tables below 4 GB are addressed with 32-bit offsets - rows of up to
 *     128 bytes with a shift, wider ones, below 2^24 vertices, with a 24-bit multiply - larger ones
 *     with 64-bit loads),
 * and otherwise runs the group kernel over the same plan.  A plan that contains empty groups has no
 * stream form.  No counterpart in the reference.
 *
 * Life of a plan.  The plan's memory is the caller's; the library remembers, by the plan's address, the
 * header it read in eppgcn_plan_status (counts and the number of the build).  Tell it with
 * eppgcn_plan_release before that memory is freed or reused, and rebuild a plan whose bytes were
 * overwritten.  The stream and fix-up kernels compare the header in memory with the remembered one before
 * they index anything: on a difference they write no output and leave a mark, which
 * eppgcn_aggregation_status reports as EPPGCN_ERR_PLAN_MISMATCH (the aggregation calls themselves are
 * asynchronous and cannot). */
/* 1 when a plan is expected to pay off: the [num_nodes, dim] feature table has 4 MB or more.  Large
 * tables (hundreds of MB) gain from the column-blocked order; small ones still gain from the
 * length-sorted groups, the precomputed group flags and the selective output clear; below that the
 * calls are launch-bound and a plan changes nothing. */
int eppgcn_plan_recommended(int64_t num_nodes, int dim);
size_t eppgcn_plan_bytes(int64_t num_parts, int64_t num_slots, int64_t num_nodes);
size_t eppgcn_plan_workspace_bytes(int64_t num_parts, int64_t num_slots);
int eppgcn_build_plan(const int32_t* part_pointers, const int32_t* column_index,
                      const int32_t* part2node, const int32_t* ids, int num_parts, int64_t num_slots,
                      int num_nodes, int dim, int block_shift, void* plan, size_t plan_bytes,
                      void* workspace, size_t workspace_bytes, void* stream);
/* eppgcn_build_plan is asynchronous and contains look-back scans.  This call synchronises `stream`,
 * reads the plan's header and returns 0, EPPGCN_ERR_SCAN_STALLED (a stalled scan leaves a corrupt
 * plan, which must not be used) or EPPGCN_ERR_PLAN_MISMATCH (the memory does not hold the header of a
 * finished build of this process with these sizes).  Pass the sizes the plan was built with.  *partial_rows (may be
 * NULL) receives the number of partial sums a call through the stream form needs room for (0 when
 * the plan has no stream form).  The library remembers the header by the plan's address until the
 * next eppgcn_build_plan into that address, and the aggregation calls use the stream form only for
 * plans it knows this way: call it once after the build (the build's workspace may be released
 * afterwards); a plan copied to another address runs through the group kernel until this has been
 * called for the copy. */
int eppgcn_plan_status(const void* plan, int num_parts, int64_t num_slots, int num_nodes,
                       int64_t* partial_rows, void* stream);
/* Makes the library forget what it remembers about the plan at this address (NULL is ignored).  Call it
 * before the plan's memory is freed or reused; eppgcn_build_plan into the same address does it by itself. */
void eppgcn_plan_release(const void* plan);
/* Synchronises `stream` and returns EPPGCN_ERR_PLAN_MISMATCH - once - when, since the last such report,
 * the stream or fix-up kernel of an aggregation call on the current device found a plan header in memory
 * that was not the one eppgcn_plan_status had read at that address (the plan's bytes were overwritten, or
 * its memory was reused without eppgcn_plan_release).  That call wrote no output.  0 otherwise.  Ask once
 * per batch of calls, next to the other status calls; planned calls through the group kernel and calls
 * without a plan never raise it. */
int eppgcn_aggregation_status(void* stream);
/* Floats of the feature workspace that lets a [num_nodes, dim] aggregation over `plan` take the
 * stream form: eppgcn_feature_workspace_floats(num_nodes, dim) plus one row per partial sum (what
 * eppgcn_plan_status reported).  Equal to eppgcn_feature_workspace_floats for NULL or a plan
 * without (known) stream form. */
size_t eppgcn_plan_workspace_floats(const void* plan, int64_t num_nodes, int dim);
/* 1 when the calling thread's last aggregation call ran the stream form, 0 when it ran the group kernel. */
int eppgcn_last_call_used_stream(void);

/* Forward neighbour-group aggregation:
 *   out[r,:] = sum_{e in groups of r} fl32(degrees[r]*degrees[col[e]]) * in[col[e],:]
 * `out` ([num_nodes, dim]) is fully overwritten (rows without groups become 0).
 * Stands in for spmm_forward_cuda minus its torch::mm (EPPGCN_kernel.cu:123-202;
 * kernel :204-295; bound as GNNA.forward, EPPGCN.cpp:79-102,390).  row_pointers
 * may be NULL (the reference's kernel never reads it).  part_size, dim_worker and
 * warp_per_block are the caller's launch hints for 32-lane warps; the wave64
 * mapping is chosen from `dim`, the hints only have to be positive. */
int eppgcn_spmm_forward(float* out, const float* in, const int32_t* row_pointers,
                        const int32_t* column_index, const float* degrees,
                        const int32_t* part_pointers, const int32_t* part2node,
                        int num_nodes, int dim, int num_parts,
                        int part_size, int dim_worker, int warp_per_block,
                        float* workspace, size_t workspace_floats, const void* plan, void* stream);

/* Unpruned backward aggregation: the same operator applied to d_output (valid
 * because the normalised adjacency is symmetric).  Stands in for
 * spmm_backward_cuda minus its two torch::mm (EPPGCN_kernel.cu:395-469; kernel
 * :471-545; bound as GNNA.backward, EPPGCN.cpp:104-130,391). */
int eppgcn_spmm_backward(float* d_input, const float* d_output, const int32_t* row_pointers,
                         const int32_t* column_index, const float* degrees,
                         const int32_t* part_pointers, const int32_t* part2node,
                         int num_nodes, int dim, int num_parts,
                         int part_size, int dim_worker, int warp_per_block,
                         float* workspace, size_t workspace_floats, const void* plan, void* stream);

/* Pruned backward aggregation over the compacted execution path:
 *   d_input[id_p,:] += sum_{k in group p} fl32(degrees[id_p]*degrees[edge_list[k]]) * d_output[edge_list[k],:]
 * with id_p = ids[part_pointer[p]]; d_input is fully overwritten (zero elsewhere).
 * part_pointer holds num_parts+1 entries.  Stands in for ours_backward_cuda minus
 * its two torch::mm (EPPGCN_kernel.cu:547-624; kernel :626-670; bound as
 * GNNA.ours_backward, EPPGCN.cpp:157-184,393).  `layer` (1-based) only selects the
 * per-layer timer; blockx/blocky are the caller's hints and must be positive.
 * gathered_rows: NULL, or the bitmap eppgcn_mark_gathered_rows made of this edge_list; the
 * pre-scaling pass into the workspace then skips the rows of d_output that no group reads (with a
 * 10 % train mask the last layer's path reads a tenth of the rows), which changes no result; with
 * the workspace aliasing d_output, only those rows of d_output are overwritten with scaled values. */
int eppgcn_ours_backward(float* d_input, const float* d_output, const int32_t* ids,
                         const int32_t* part_pointer, const int32_t* edge_list, const float* degrees,
                         int num_nodes, int dim, int num_parts, int part_size, int layer,
                         int blockx, int blocky, float* workspace, size_t workspace_floats, const void* plan,
                         const uint32_t* gathered_rows, void* stream);
/* eppgcn_ours_backward for a caller that reads d_input only in the rows the path writes (the dense products
 * of the layer's backward step, eppgcn_update_backward_rows): the same call, same results in those rows, but
 * when it runs a plan's stream form the rows without any group are LEFT AS THEY ARE instead of being cleared
 * (with a 10 % train mask two thirds of the rows of the last layer's gradient: the clear was most of a heavily
 * pruned call), and *written_rows receives the device address of the bitmap of the rows that were written
 * (bit r of word r / 32; it lies inside the plan and lives as long as the plan), *num_written (may be NULL)
 * their number.  When the call cannot skip the clear (no plan, no stream form for the shape or workspace),
 * it clears as eppgcn_ours_backward does and sets *written_rows = NULL: every row of d_input is defined.
 * The reference sketches the consumer side of this in the comments of ours_backward_cuda
 * (`X.index({mask})`, EPPGCN_kernel.cu:607,616); it has no such call itself. */
int eppgcn_ours_backward_rows(float* d_input, const float* d_output, const int32_t* ids,
                              const int32_t* part_pointer, const int32_t* edge_list, const float* degrees,
                              int num_nodes, int dim, int num_parts, int part_size, int layer,
                              int blockx, int blocky, float* workspace, size_t workspace_floats, const void* plan,
                              const uint32_t* gathered_rows, const uint32_t** written_rows, int64_t* num_written,
                              void* stream);

/* bitmap[(num_nodes + 31) / 32]: bit c is set for every vertex c that occurs in
 * edge_list[0 .. valid_len) (the rows a pruned backward over this path gathers); *d_count (device)
 * and, if not NULL, *h_count (host; synchronises the stream) receive the number of such vertices.
 * Built once per path, next to the path itself.  No counterpart in the reference. */
int eppgcn_mark_gathered_rows(const int32_t* edge_list, int64_t valid_len, int num_nodes, uint32_t* bitmap,
                              int32_t* d_count, int64_t* h_count, void* stream);

/* ---------------------------------------------------------------------------
 * Execution-path preparation.
 * ------------------------------------------------------------------------- */

/* Marks one layer's backward path from the forward groups (in place):
 *   slot e of row r with src_mask[col[e]]      -> back_edge_mask[e] = r, node_degs[r] += 1
 *   !is_last_layer and src_mask[r]             -> ngh_mask[r] = ngh_mask[col[e]] = 1
 * back_edge_mask must be pre-filled with -1 and node_degs with 0 by the caller
 * (EPPGCN/dataset.py:149-156); ngh_mask may be NULL when is_last_layer.  Stands in
 * for mask_forward_cuda (EPPGCN_kernel.cu:297-349; kernel :351-388; bound as
 * GNNA.mask_forward, EPPGCN.cpp:132-155,392; is_last_layer = (layer == num_layers)). */
int eppgcn_mask_forward(const int32_t* part2node, const int32_t* part_pointers,
                        const int32_t* column_index, const uint8_t* src_mask, uint8_t* ngh_mask,
                        int32_t* back_edge_mask, int32_t* node_degs, int num_parts,
                        int64_t num_edges, int is_last_layer, int blockx, int blocky, void* stream);

/* Workspace sizes for the scan-based functions below. */
size_t eppgcn_compact_workspace_bytes(int64_t length);
size_t eppgcn_split_workspace_bytes(int64_t num_nodes);

/* Status of the last scan-based call that used `workspace` (eppgcn_compact_back_edge,
 * eppgcn_mark_compact, eppgcn_split_back_part, eppgcn_build_part; NULL = the static scratch of
 * eppgcn_compact_back_edge_static on the current device): synchronises `stream`, then
 * returns 0, EPPGCN_ERR_SCAN_STALLED (a look-back wait hit its spin limit: the outputs of that call
 * are invalid) or EPPGCN_ERR_CAPACITY (the group pointers did not fit).  The scan-based calls check
 * this themselves only when a host result (h_*) is requested; a caller that takes every count on
 * the device (all h_* NULL) gets return code 0 from them whatever happened on the device and must
 * call this once before it trusts the outputs. */
int eppgcn_scan_status(const void* workspace, void* stream);

/* Stable two-array compaction of the slots with edge_mask[e] != -1:
 *   out_id[k] = edge_mask[e_k], out_edge[k] = column_index[e_k], k < V; both
 * outputs (length entries each) are zero from V on.  V is left in device memory at
 * d_valid_len (may be NULL) and, when h_valid_len is not NULL, copied to the host
 * after synchronising.  Stands in for compact_mask (cuCompactor.cu:682-686 over
 * :328-465) as compact_back_edge uses it (EPPGCN.cpp:282-296,399). */
int eppgcn_compact_back_edge(const int32_t* edge_mask, const int32_t* column_index,
                             int32_t* out_id, int32_t* out_edge, int64_t length,
                             void* workspace, size_t workspace_bytes,
                             int32_t* d_valid_len, int64_t* h_valid_len, void* stream);

/* eppgcn_compact_back_edge for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): same inputs, outputs and results,
 * but the scan scratch is a static device array inside the library instead of a caller workspace,
 * and the call allocates nothing (no hipMalloc / hipFree, no allocating library routine).  No
 * counterpart in the reference, whose compactor allocates and frees its scratch on every call
 * (cuCompactor.cu:328-465).
 *   - length may be at most eppgcn_compact_back_edge_static_max_length() = 2^30 slots; a longer
 *     input fails with EPPGCN_ERR_CAPACITY and a message, before any device work.
 *   - The array (512 KiB + 32 bytes: the scan state and one descriptor per 16384-slot tile) exists once
 *     per GPU the library runs on, for the life of the process; its address on a device is looked up on
 *     the first call there (the device that is current at the call).  A caller that captures the call
 *     into a HIP graph makes one call - this one, or eppgcn_scan_status(NULL, stream) - on that device
 *     outside the capture first.
 *   - With h_valid_len == NULL nothing synchronises and a stalled look-back goes unreported by the call
 *     itself: eppgcn_scan_status(NULL, stream) reads the status from the static scratch afterwards.
 *   - Every call on a GPU uses that GPU's one array (it is cleared at the start of each call), so
 *     calls that overlap on one GPU - on different streams or from different threads - race and
 *     must be serialised by the caller. */
int64_t eppgcn_compact_back_edge_static_max_length(void);
int eppgcn_compact_back_edge_static(const int32_t* edge_mask, const int32_t* column_index,
                                    int32_t* out_id, int32_t* out_edge, int64_t length,
                                    int32_t* d_valid_len, int64_t* h_valid_len, void* stream);

/* Path marking and compaction of one layer in one pass over the slots: exactly the results of
 * eppgcn_mask_forward on a -1-filled edge mask followed by eppgcn_compact_back_edge (ngh_mask and
 * node_degs updated in place, out_id / out_edge with zero tails, V at d_valid_len / h_valid_len),
 * without the num_edges-entry edge mask in between.  The reference runs the two steps separately
 * (mask_forward_cuda, EPPGCN_kernel.cu:297-388, inside the first forward; compact_mask,
 * cuCompactor.cu:328-465, from gcn_main.py:154); this call is for drivers that prepare the path
 * before training.  The groups must tile the slots in order, as build_part produces them.
 * workspace: eppgcn_mark_compact_workspace_bytes(num_edges) bytes, 8-byte aligned. */
size_t eppgcn_mark_compact_workspace_bytes(int64_t num_edges);
int eppgcn_mark_compact(const int32_t* part2node, const int32_t* part_pointers,
                        const int32_t* column_index, const uint8_t* src_mask, uint8_t* ngh_mask,
                        int32_t* node_degs, int32_t* out_id, int32_t* out_edge, int num_parts,
                        int64_t num_edges, int is_last_layer, void* workspace, size_t workspace_bytes,
                        int32_t* d_valid_len, int64_t* h_valid_len, void* stream);

/* Number of entries != 0 (valid_node of the group-size heuristics).  Stands in for
 * compact_count (cuCompactor.cu:694-696 over :623-680).  d_count: one device int. */
int eppgcn_count_nonzero(const int32_t* node_deg, int64_t length, int32_t* d_count,
                         int64_t* h_count, void* stream);

/* Backward group size from the fitted regression, in double arithmetic with C
 * round() (EPPGCN.cpp:303-310, get_map_back_part_size).  Pure host function.
 * The raw value can be <= 0 on large sparse paths; *clamped (may be NULL) is set
 * when the returned value was raised to 1. */
int eppgcn_map_back_part_size(int64_t valid_node, int64_t valid_len, int* clamped);
/* Legacy threshold rule of build_back_part (EPPGCN.cpp:246-258); returns 0 when the
 * ratio is >= 512, as the reference leaves it. */
int eppgcn_threshold_back_part_size(int64_t valid_node, int64_t valid_len);
/* The same decision re-fitted for the wave64 kernels of this library: 16 while the path keeps fewer
 * than 24 edges per row with kept edges, 32 above.  With partial sums carried from group to group
 * inside a wave the group size matters far less than for the reference's kernel (within 10 % over
 * 8..64 in every measured cell), so two values are all the fit supports.  No counterpart in the
 * reference (its rules are EPPGCN.cpp:246-258 and :303-310). */
int eppgcn_wave64_back_part_size(int64_t valid_node, int64_t valid_len);

/* The group size a caller of the reference's `map` mode should use with this library: the fitted
 * regression (eppgcn_map_back_part_size) while it yields at least 1, otherwise - on large paths,
 * where the regression, which was fitted on small graphs, goes negative (-143 at 10^6 rows with 10^8
 * kept edges) - the wave64 rule above instead of a clamp to 1 (which would cut a path of 10^8 kept
 * edges into 10^8 one-slot groups).  *fell_back (may be NULL) is set when the wave64 rule was used.
 * Stands in for get_map_back_part_size (EPPGCN.cpp:298-325) in drivers. */
int eppgcn_auto_back_part_size(int64_t valid_node, int64_t valid_len, int* fell_back);

/* Splits the kept edges of every vertex into groups of part_size and writes the
 * group pointers: part_pointer[0..P] with part_pointer[P] = V, zero after that up
 * to `capacity` entries.  d_counts (may be NULL) receives {P, V} on the device;
 * h_num_parts / h_valid_len are filled after synchronising when not NULL.
 * Fails with EPPGCN_ERR_CAPACITY (host results requested) if P + 1 > capacity.
 * Stands in for compact_part + exclusive_scan (cuCompactor.cu:688-692 over
 * :467-621, and :42-48) as split_back_part composes them (EPPGCN.cpp:327-346,401). */
int eppgcn_split_back_part(const int32_t* node_deg, int num_nodes, int part_size,
                           int32_t* part_pointer, int64_t capacity,
                           void* workspace, size_t workspace_bytes, int32_t* d_counts,
                           int64_t* h_num_parts, int64_t* h_valid_len, void* stream);

/* Forward neighbour groups from the CSR row pointers (device): part_pointers[0..P]
 * (terminator = row_pointers[num_nodes]) and part2node[0..P-1]; `capacity` is the
 * number of entries part_pointers can hold (part2node: capacity - 1); an upper
 * bound is num_edges / part_size + num_nodes + 1.  Stands in for build_part
 * (EPPGCN.cpp:186-227,397), which the reference runs on the CPU. */
int eppgcn_build_part(const int32_t* row_pointers, int num_nodes, int part_size,
                      int32_t* part_pointers, int32_t* part2node, int64_t capacity,
                      void* workspace, size_t workspace_bytes, int32_t* d_counts,
                      int64_t* h_num_parts, void* stream);

/* Degree-distribution features of get_ginfo (EPPGCN.cpp:348-386,402): h_out[10]
 * on the host; d_hist: ten device ints of scratch.  Synchronises. */
int eppgcn_get_ginfo(const int32_t* node_deg, int64_t num_nodes, int64_t valid_len,
                     int32_t* d_hist, float* h_out, void* stream);

/* ---------------------------------------------------------------------------
 * Dense update of a layer: the matrix products the reference computes with torch::mm around
 * the aggregation, for tall-and-skinny shapes (num_nodes rows, tens of columns), on the fp32
 * matrix cores.  All matrices are fp32 row-major and contiguous unless a pitch is given.
 * A call fails with EPPGCN_ERR_INVALID_ARGUMENT (and a message) for shapes outside what the
 * kernels cover (reduction length beyond 1024, more than 64 gradient columns for the weight
 * gradient); callers then use a general GEMM.
 * ------------------------------------------------------------------------- */

/* Bit mask of the update functions that cover [*, in_dim] x [in_dim, out_dim] layers:
 * 1 eppgcn_update_forward, 2 eppgcn_update_backward_input, 4 eppgcn_update_backward_weight. */
int eppgcn_update_supported(int in_dim, int out_dim);

/* out[r, 0:out_dim] = scale[r] * act(x[r, :]) * w, columns out_dim..ld_out-1 = 0.
 * x [num_nodes, in_dim], w [in_dim, out_dim], out rows ld_out floats apart; scale may be NULL
 * (factor 1); relu_input != 0 applies max(x, 0) on load.
 * Replaces `tmp = torch::mm(input, weight)`, EPPGCN_kernel.cu:142 (spmm_forward_cuda). */
int eppgcn_update_forward(float* out, int ld_out, const float* x, const float* w, const float* scale,
                          int relu_input, int64_t num_nodes, int in_dim, int out_dim, void* stream);
/* The same product written as the pre-scaled feature workspace the aggregation functions accept with a
 * NULL input: table[eppgcn_feature_workspace_row(r), :] = scale[r] * act(x[r, :]) * w, rows
 * eppgcn_feature_workspace_pitch(out_dim) floats apart with zeros in the padding; `table` holds
 * table_floats >= eppgcn_feature_workspace_floats(num_nodes, out_dim) floats (more when partial sums follow
 * it, see eppgcn_plan_workspace_floats), 16-byte aligned.  No separate scaling pass is then needed. */
int eppgcn_update_forward_table(float* table, size_t table_floats, const float* x, const float* w,
                                const float* scale, int relu_input, int64_t num_nodes, int in_dim,
                                int out_dim, void* stream);

/* d_x[num_nodes, in_dim] = g[num_nodes, out_dim] * w^T, w [in_dim, out_dim]; with relu_ref
 * ([num_nodes, in_dim], may be NULL) entries where relu_ref <= 0 are zeroed (gradient of a
 * ReLU applied to the layer input).
 * Replaces `d_input = torch::mm(d_input_prime, W.transpose(0,1))`, EPPGCN_kernel.cu:461,614. */
int eppgcn_update_backward_input(float* d_x, const float* g, const float* w, const float* relu_ref,
                                 int64_t num_nodes, int in_dim, int out_dim, void* stream);

/* d_w[in_dim, out_dim] = act(x)^T * g, x [num_nodes, in_dim], g [num_nodes, out_dim], out_dim <= 64.
 * Sums are formed in a fixed order (bitwise reproducible).  workspace: at least
 * eppgcn_update_workspace_bytes(num_nodes, in_dim, out_dim) bytes, 4-byte aligned.
 * Replaces `d_weight = torch::mm(X.transpose(0,1), d_input_prime)`, EPPGCN_kernel.cu:462,615. */
size_t eppgcn_update_workspace_bytes(int64_t num_nodes, int in_dim, int out_dim);
int eppgcn_update_backward_weight(float* d_w, const float* x, const float* g, int relu_input, int64_t num_nodes,
                                  int in_dim, int out_dim, void* workspace, size_t workspace_bytes, void* stream);

/* Both gradients of a layer out = act(x) * w in one call: d_x as eppgcn_update_backward_input gives it with
 * relu_ref = x when relu_input != 0 (NULL otherwise), d_w as eppgcn_update_backward_weight gives it - the same
 * bits.  For narrow layers (in_dim <= 16, out_dim <= 32) one kernel forms both products from one pass over x
 * and g (they come from memory once instead of twice); other shapes run the two kernels one after the other
 * and are subject to their limits (out_dim <= 64).  workspace as for eppgcn_update_backward_weight.
 * Replaces the pair `d_input = torch::mm(d_input_prime, W.transpose(0,1))`, `d_weight =
 * torch::mm(X.transpose(0,1), d_input_prime)`, EPPGCN_kernel.cu:461-462,614-615. */
int eppgcn_update_backward(float* d_x, float* d_w, const float* x, const float* g, const float* w, int relu_input,
                           int64_t num_nodes, int in_dim, int out_dim, void* workspace, size_t workspace_bytes,
                           void* stream);
/* eppgcn_update_backward for a gradient of which only some rows are defined: `rows` holds one bit per row of g
 * (bit r of word r / 32, (num_nodes + 31) / 32 words; NULL = every row, i.e. eppgcn_update_backward).  A row whose
 * bit is clear counts as zeros and is not read - neither that row of g, which may hold anything, nor the row of x
 * it would be multiplied with; its row of d_x is written as zeros.  Where the rows with clear bits do hold zeros (and
 * finite values in x) the results equal those of eppgcn_update_backward bit for bit.  d_x may be NULL (and then w): only d_w is formed (a
 * first layer whose input needs no gradient).  This is the row-masked product the reference sketches in
 * `d_weight = torch::mm(X.index({mask}).transpose(0,1), d_input_prime.index({mask}))`, EPPGCN_kernel.cu:616, taken
 * over the bitmap eppgcn_ours_backward_rows hands out instead of an index list. */
int eppgcn_update_backward_rows(float* d_x, float* d_w, const float* x, const float* g, const float* w, int relu_input,
                                const uint32_t* rows, int64_t num_nodes, int in_dim, int out_dim, void* workspace,
                                size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------
 * Timers (print_time / clear_time, EPPGCN_kernel.cu:89-116; EPPGCN.cpp:394-395).
 * Timing is off by default so that calls stay asynchronous; when enabled every
 * aggregation / marking call brackets its kernels with events and synchronises.
 * Not thread-safe, like the reference's file-scope accumulators.
 * ------------------------------------------------------------------------- */
void eppgcn_set_timing(int enabled);
void eppgcn_print_time(void);
void eppgcn_clear_time(void);
/* which: 0 forward aggregation, 1 backward aggregation (all layers), 2 path marking,
 * 3 the output clears and 4 the pre-scaling passes of the aggregation calls (0 and 1 cover the
 * aggregation kernels alone, as the reference's timers do), 100+k backward aggregation of layer k
 * (1-based, k <= 16).  Milliseconds. */
double eppgcn_get_time_ms(int which);

#ifdef __cplusplus
}
#endif
#endif /* EPPGCN_HIP_H_ */
