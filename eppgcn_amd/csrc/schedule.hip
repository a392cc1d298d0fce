// Column-blocked execution plan for the aggregation kernels.
//
// The aggregation gathers feature rows at random; in CSR row order the rows gathered at any
// moment are spread over the whole table and two thirds of the gathers go to HBM.  A plan is a
// copy of the groups re-ordered by the column block of their first slot (blocks of 2^shift
// vertices, original order inside a block): the waves in flight then work on one window of
// columns whose rows are served from L2.  The plan holds everything the kernel reads per group
// in processing order, so that all of it streams:
//
//     ptr[P+1]   slot offsets into `col`            row[P]    row of the group
//     flags[P]   bit0 the row has groups before this one (original order), bit1 after it,
//                bit2 this group continues the previous plan entry (same row, next original
//                index), bit3 the next plan entry continues this one
//     col[S]     column ids, group by group in plan order
//     single[ceil(N/32)]  bit r set: row r has exactly one group and the group is not empty; the
//                kernel writes such a row with one plain store, so the output clear can skip it
//
// The re-ordering changes no result, only which groups run together.  It depends on the graph
// and the groups alone: a caller builds it once and passes it to every aggregation call.
//
// The stable sort of (block, group index) pairs is rocPRIM's device radix sort, a library
// routine in a preparation step, as the reference uses thrust for its scans; everything else
// (keys, look-back scan of the group sizes, flags, column copy) is written here.
#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>

#include "common.hpp"

namespace eppgcn {

static size_t align256(size_t x) { return (x + 255) / 256 * 256; }

// ---------------------------------------------------------------- kernels
// Sort key of group p: the column block of its first slot, except that all groups of a short row
// (at most `keep_slots` slots in at most kMaxRowWalk groups) share the key of the row's first group:
// such a row stays together in the plan, is summed in registers and written once with plain stores,
// instead of leaving one partial sum per column block to be combined with atomics (measured at group
// size 31: the atomics of rows with 2..16 groups cost more than the L2 hits of their later groups
// save; the bound is in slots because a row's gathers, not its groups, are what a block can speed up:
// with groups of 4-8 slots a bound in groups spread rows of 40 slots and lost up to 2x at 256 columns).
constexpr int kMaxRowWalk = 64;
__global__ __launch_bounds__(256) void plan_keys_kernel(const int* __restrict__ part_ptr, const int* __restrict__ col,
                                                       const int* __restrict__ part2node, const int* __restrict__ ids,
                                                       int num_parts, int shift, int keep_slots, int classes,
                                                       unsigned* __restrict__ keys, int* __restrict__ iota)
{
    const int p = blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= num_parts) return;
    iota[p] = p;
    const int beg = part_ptr[p];
    const int end = part_ptr[p + 1];
    if (end <= beg) { keys[p] = 0u; return; }
    const int row = part2node ? part2node[p] : ids[beg];
    auto same_row = [&](int j) {
        const int b = part_ptr[j];
        if (part_ptr[j + 1] <= b) return false;
        return (part2node ? part2node[j] : ids[b]) == row;
    };
    int start = p;
    for (int k = 0; k < kMaxRowWalk && start > 0 && same_row(start - 1); ++k) --start;
    const bool start_found = !(start > 0 && same_row(start - 1));
    int last = p;
    while (last + 1 < num_parts && last + 1 - start < kMaxRowWalk && same_row(last + 1)) ++last;
    const bool end_found = !(last + 1 < num_parts && same_row(last + 1));
    const bool short_row = keep_slots > 0 && start_found && end_found && last - start + 1 <= kMaxRowWalk &&
                           part_ptr[last + 1] - part_ptr[start] <= keep_slots;
    const int key_col = short_row ? col[part_ptr[start]] : col[beg];
    unsigned key = static_cast<unsigned>(key_col) >> shift;
    if (classes) {
        // second key: length class of a row that is a single group (a class = one gather step of 8
        // slots), so that the groups a wave works on in one round take the same number of steps;
        // rows of several groups consist of full groups but for the last one: class 3
        const int len = end - beg;
        const int cls = (short_row && start == last) ? min(3, (len - 1) >> 3) : 3;
        key = (key << 2) | static_cast<unsigned>(cls);
    }
    keys[p] = key;
}

__global__ __launch_bounds__(256) void plan_sizes_kernel(const int* __restrict__ part_ptr, const int* __restrict__ order,
                                                        int num_parts, int* __restrict__ sizes)
{
    const int q = blockIdx.x * blockDim.x + threadIdx.x;
    if (q >= num_parts) return;
    const int p = order[q];
    sizes[q] = part_ptr[p + 1] - part_ptr[p];
}

// Exclusive prefix sum of `in[0..n)` into `out[0..n]` (out[n] = total): single pass, decoupled
// look-back over tiles of 2048.
constexpr int kScanBlock = 256;
constexpr int kScanItems = 8;
constexpr int kScanTile = kScanBlock * kScanItems;

__global__ __launch_bounds__(kScanBlock) void exclusive_scan_kernel(const int* __restrict__ in, int* __restrict__ out,
                                                                   int n, int num_tiles, ScanState* st, uint64_t* desc)
{
    __shared__ int s_tile;
    __shared__ int s_wave[kScanBlock / kWave];
    __shared__ int s_excl;
    const int tile = acquire_tile(st, &s_tile);
    if (tile >= num_tiles) return;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const long long base = static_cast<long long>(tile) * kScanTile + threadIdx.x * kScanItems;
    int v[kScanItems];
    int sum = 0;
#pragma unroll
    for (int j = 0; j < kScanItems; ++j) {
        v[j] = base + j < n ? in[base + j] : 0;
        sum += v[j];
    }
    const int incl = wave_inclusive_scan(sum);
    if (lane == kWave - 1) s_wave[wave] = incl;
    __syncthreads();
    int wave_excl = 0, total = 0;
#pragma unroll
    for (int w = 0; w < kScanBlock / kWave; ++w) {
        if (w < wave) wave_excl += s_wave[w];
        total += s_wave[w];
    }
    if (wave == 0) {
        const uint64_t excl = tile_lookback(desc, st, tile, static_cast<uint64_t>(total));
        if (lane == 0) s_excl = static_cast<int>(excl);
    }
    __syncthreads();
    int run = s_excl + wave_excl + incl - sum;
#pragma unroll
    for (int j = 0; j < kScanItems; ++j) {
        if (base + j < n) out[base + j] = run;
        run += v[j];
    }
    if (tile == num_tiles - 1 && threadIdx.x == kScanBlock - 1) out[n] = run;
}

// row, flags and the column copy of every plan entry; a team of 8 lanes per group.
__global__ __launch_bounds__(256) void plan_fill_kernel(const int* __restrict__ part_ptr, const int* __restrict__ col,
                                                       const int* __restrict__ part2node, const int* __restrict__ ids,
                                                       const int* __restrict__ order, int num_parts, PlanView plan)
{
    constexpr int kTeam = 8;
    const long long t = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    const long long q = t / kTeam;
    const int tl = static_cast<int>(t % kTeam);
    if (q >= num_parts) return;
    const int p = order[q];
    const int beg = part_ptr[p];
    const int end = part_ptr[p + 1];
    const int dst = plan.ptr[q];
    for (int i = tl; i < end - beg; i += kTeam) plan.col[dst + i] = col[beg + i];
    if (tl == 0) {
        int row = 0;
        bool prev = false, next = false;
        if (end > beg) {
            if (part2node) {
                row = part2node[p];
                prev = p > 0 && part2node[p - 1] == row;
                next = p + 1 < num_parts && part2node[p + 1] == row;
            } else {
                row = ids[beg];
                prev = beg > 0 && ids[beg - 1] == row;
                next = p + 1 < num_parts && ids[end] == row;
            }
        }
        const bool joins_left = prev && q > 0 && order[q - 1] == p - 1;
        const bool joins_right = next && q + 1 < num_parts && order[q + 1] == p + 1;
        if (end > beg && !prev && !next) atomicOr(plan.single + (row >> 5), 1u << (row & 31));
        plan.row[q] = row;
        plan.flags[q] = static_cast<uint8_t>((prev ? 1 : 0) | (next ? 2 : 0) | (joins_left ? 4 : 0) | (joins_right ? 8 : 0));
    }
}

// ---------------------------------------------------------------- host
static hipError_t sort_temp_bytes(int num_parts, int bits, size_t* bytes)
{
    *bytes = 0;
    return rocprim::radix_sort_pairs(nullptr, *bytes, static_cast<unsigned*>(nullptr), static_cast<unsigned*>(nullptr),
                                     static_cast<int*>(nullptr), static_cast<int*>(nullptr),
                                     static_cast<size_t>(num_parts), 0u, static_cast<unsigned>(bits));
}

static size_t scan_state_bytes(long long n)
{
    const long long tiles = (n + kScanTile - 1) / kScanTile;
    return align256(sizeof(ScanState) + sizeof(uint64_t) * static_cast<size_t>(tiles > 0 ? tiles : 1));
}

// workspace layout: keys_in | keys_out | iota | order | sizes | scan state | rocPRIM temporary storage
size_t plan_workspace_bytes(long long num_parts)
{
    if (num_parts <= 0) return 256;
    size_t temp = 0;
    if (sort_temp_bytes(static_cast<int>(num_parts), 32, &temp) != hipSuccess) temp = 0;
    return 5 * align256(sizeof(int) * (static_cast<size_t>(num_parts) + 1)) + scan_state_bytes(num_parts) +
           align256(temp) + 256;
}

// where launch_build_plan keeps the state of its look-back scan inside the workspace
size_t plan_scan_state_offset(long long num_parts)
{
    return 5 * align256(sizeof(int) * (static_cast<size_t>(num_parts > 0 ? num_parts : 0) + 1));
}

int workspace_pitch(int dim);   // aggregate.hip

static int g_force_shift = 0;
static int g_keep_rows = 8;      // in units of 32 slots: rows of up to 256 slots stay together
static int g_length_classes = 1;
void set_plan_length_classes(int on) { g_length_classes = on ? 1 : 0; }
void set_schedule_shift(int shift) { g_force_shift = shift; }
void set_plan_keep_rows(int keep) { g_keep_rows = keep < 0 ? 0 : keep; }

int schedule_shift(int dim)
{
    if (g_force_shift > 0) return g_force_shift;
    // column blocks of at most 128K rows and 16 MB of feature rows.  Measured at R-MAT scale 22
    // (ms per epoch, 64- and 128-byte rows): 2^14 5.95, 2^15 5.74, 2^16 5.63, 2^17 5.60, 2^18 5.65,
    // 2^19 5.83 - the window all waves gather from has to stay resident in the memory-side cache,
    // not in one XCD's L2, and larger blocks leave fewer partial sums to combine
    const int row_bytes = 4 * workspace_pitch(dim);
    int shift = 17;
    while (shift > 8 && (static_cast<long long>(row_bytes) << shift) > (16ll << 20)) --shift;
    return shift;
}

__global__ void plan_scan_init_kernel(ScanState* st, uint64_t* desc, int num_tiles)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < num_tiles) desc[i] = kTileEmpty;
    if (i == 0) {
        st->counter = 0;
        st->error = 0;
        st->counts[0] = st->counts[1] = 0;
        st->overflow = 0;
    }
}

int launch_build_plan(const int* part_ptr, const int* col, const int* part2node, const int* ids, int num_parts,
                      long long num_slots, int num_nodes, int shift, void* plan, size_t plan_size, void* workspace,
                      size_t workspace_bytes, hipStream_t stream)
{
    if (num_parts <= 0) return kOk;
    if (plan_size < plan_bytes(num_parts, num_slots, num_nodes)) {
        set_error("build_plan: plan buffer smaller than eppgcn_plan_bytes(num_parts, num_slots, num_nodes)");
        return kErrInvalidArgument;
    }
    const size_t slab = align256(sizeof(int) * (static_cast<size_t>(num_parts) + 1));
    char* base = static_cast<char*>(workspace);
    unsigned* keys_in = reinterpret_cast<unsigned*>(base);
    unsigned* keys_out = reinterpret_cast<unsigned*>(base + slab);
    int* iota = reinterpret_cast<int*>(base + 2 * slab);
    int* order = reinterpret_cast<int*>(base + 3 * slab);
    int* sizes = reinterpret_cast<int*>(base + 4 * slab);
    ScanState* st = reinterpret_cast<ScanState*>(base + plan_scan_state_offset(num_parts));
    uint64_t* desc = reinterpret_cast<uint64_t*>(st + 1);
    void* temp = base + 5 * slab + scan_state_bytes(num_parts);
    int bits = 1;
    while (bits < 30 && (static_cast<long long>(num_nodes) >> shift) >= (1ll << bits)) ++bits;
    if (g_length_classes) bits += 2;
    size_t temp_bytes = 0;
    EPPGCN_HIP(sort_temp_bytes(num_parts, bits, &temp_bytes));
    if (5 * slab + scan_state_bytes(num_parts) + temp_bytes > workspace_bytes) {
        set_error("build_plan: workspace smaller than eppgcn_plan_workspace_bytes(num_parts)");
        return kErrInvalidArgument;
    }
    const unsigned blocks = static_cast<unsigned>((num_parts + 255) / 256);
    hipLaunchKernelGGL(plan_keys_kernel, dim3(blocks), dim3(256), 0, stream, part_ptr, col, part2node, ids, num_parts,
                       shift, g_keep_rows * 32, g_length_classes, keys_in, iota);
    EPPGCN_HIP(hipGetLastError());
    EPPGCN_HIP(rocprim::radix_sort_pairs(temp, temp_bytes, keys_in, keys_out, iota, order,
                                         static_cast<size_t>(num_parts), 0u, static_cast<unsigned>(bits), stream));
    hipLaunchKernelGGL(plan_sizes_kernel, dim3(blocks), dim3(256), 0, stream, part_ptr, order, num_parts, sizes);
    EPPGCN_HIP(hipGetLastError());
    const int tiles = (num_parts + kScanTile - 1) / kScanTile;
    hipLaunchKernelGGL(plan_scan_init_kernel, dim3((tiles + 255) / 256), dim3(256), 0, stream, st, desc, tiles);
    EPPGCN_HIP(hipGetLastError());
    PlanView v = plan_view(plan, num_parts, num_nodes);
    if (int rc = launch_zero_words(v.single, plan_single_words(num_nodes), stream)) return rc;
    hipLaunchKernelGGL(exclusive_scan_kernel, dim3(tiles), dim3(kScanBlock), 0, stream, sizes, v.ptr, num_parts, tiles,
                       st, desc);
    EPPGCN_HIP(hipGetLastError());
    const long long threads = static_cast<long long>(num_parts) * 8;
    hipLaunchKernelGGL(plan_fill_kernel, dim3(static_cast<unsigned>((threads + 255) / 256)), dim3(256), 0, stream,
                       part_ptr, col, part2node, ids, order, num_parts, v);
    EPPGCN_HIP(hipGetLastError());
    return kOk;
}

}  // namespace eppgcn
