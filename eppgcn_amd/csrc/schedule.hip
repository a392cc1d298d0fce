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
// Stream form (for stream.hip).  Consecutive plan entries that continue one another form a piece (a stretch
// of slots of one row); the last slot of every piece carries bit 31 in col[], col[] is padded to a multiple
// of 512 slots with an id behind every table row (N rounded up to a multiple of 4096), and
//     erow[e]    row of piece e when the stream kernel can write it with one store (the piece is all of its row
//                and lies inside one wave's 512 slots), otherwise bit 31 | index of the partial sum it leaves
//     cev[c]     pieces that end before slot 32 c; bit 31 when slot 32 c continues a piece
//     wtail[w]   index of the partial sum for what wave w still holds at its last slot, or -1
//     touched    one bit per vertex: the row has at least one slot
//     frow/fptr  rows that have partial sums and the range of each; the partial sums are numbered row by row,
//                in stream order inside a row, so that summing a range in order gives the same bits every run
// and a header with the counts.  A plan with empty groups gets no stream form (header.valid = 0).
//
// The re-ordering changes no result, only which groups run together.  It depends on the graph
// and the groups alone: a caller builds it once and passes it to every aggregation call.
//
// Everything is written here: the keys, a stable least-significant-digit radix sort of the
// (key, group index) pairs (8 bits per pass: tile histograms, one look-back scan, stable scatter with
// ballot-based ranks), the look-back scan of the group sizes, the flags and the column copy.
#include <atomic>
#include <cstring>

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
                                                       unsigned* __restrict__ keys)
{
    const int p = blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= num_parts) return;
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
                                                                   int n, int num_tiles, ScanState* st, uint64_t* desc, unsigned mode)
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
        const uint64_t excl = tile_lookback(desc, st, tile, static_cast<uint64_t>(total), mode);
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

// ---------------------------------------------------------------- stable radix sort of (key, index) pairs
// One pass sorts by the 8-bit digit (key >> shift) & 255 and keeps the order of equal digits, so
// passes from the least significant digit upwards sort by the whole key, equal keys staying in index
// order.  A tile is kSortTile consecutive elements, element (round r, thread t) of tile T being
// T * kSortTile + r * 256 + t, so that (round, wave, lane) order is index order.
//   radix_hist_kernel     hist[d * tiles + T] = elements of tile T with digit d
//   exclusive_scan_kernel over hist (digit-major): where (digit d, tile T) starts in the output
//   radix_scatter_kernel  rank of an element among the equal digits of its wave from eight ballots,
//                         counts per (round, wave, digit) in LDS, prefix over (round, wave) per digit
constexpr int kSortBlock = 256;
constexpr int kSortRounds = 8;
constexpr int kSortTile = kSortBlock * kSortRounds;
constexpr int kDigits = 256;

__global__ __launch_bounds__(kSortBlock) void radix_hist_kernel(const unsigned* __restrict__ keys, int n, int shift,
                                                                int num_tiles, int* __restrict__ hist)
{
    __shared__ int s_hist[kDigits];
    s_hist[threadIdx.x] = 0;
    __syncthreads();
    const long long base = static_cast<long long>(blockIdx.x) * kSortTile;
#pragma unroll
    for (int r = 0; r < kSortRounds; ++r) {
        const long long i = base + r * kSortBlock + threadIdx.x;
        if (i < n) atomicAdd(&s_hist[(keys[i] >> shift) & (kDigits - 1)], 1);
    }
    __syncthreads();
    hist[static_cast<long long>(threadIdx.x) * num_tiles + blockIdx.x] = s_hist[threadIdx.x];
}

// vals_in == nullptr: the value of element i is i (first pass)
__global__ __launch_bounds__(kSortBlock) void radix_scatter_kernel(const unsigned* __restrict__ keys_in,
                                                                   const int* __restrict__ vals_in,
                                                                   unsigned* __restrict__ keys_out,
                                                                   int* __restrict__ vals_out, int n, int shift,
                                                                   int num_tiles, const int* __restrict__ offsets)
{
    constexpr int kWaves = kSortBlock / kWave;
    __shared__ int s_count[kSortRounds * kWaves][kDigits];      // per (round, wave): elements of each digit
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < kSortRounds * kWaves * kDigits; i += kSortBlock) (&s_count[0][0])[i] = 0;
    __syncthreads();
    const long long base = static_cast<long long>(blockIdx.x) * kSortTile;
    unsigned key[kSortRounds];
    int rank[kSortRounds];
#pragma unroll
    for (int r = 0; r < kSortRounds; ++r) {
        const long long i = base + r * kSortBlock + threadIdx.x;
        const bool valid = i < n;
        key[r] = valid ? keys_in[i] : 0u;
        const unsigned d = (key[r] >> shift) & (kDigits - 1);
        // lanes of the wave holding the same digit: intersect the ballots of the eight digit bits
        uint64_t peers = __ballot(valid);
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            const uint64_t set = __ballot(((d >> b) & 1u) != 0);
            peers &= ((d >> b) & 1u) ? set : ~set;
        }
        rank[r] = __popcll(peers & ((1ull << lane) - 1ull));
        if (valid && rank[r] == 0) s_count[r * kWaves + wave][d] = __popcll(peers);
    }
    __syncthreads();
    {   // thread d: exclusive prefix of digit d over the (round, wave) pairs, on top of the tile's global offset
        int run = offsets[static_cast<long long>(threadIdx.x) * num_tiles + blockIdx.x];
#pragma unroll
        for (int q = 0; q < kSortRounds * kWaves; ++q) {
            const int c = s_count[q][threadIdx.x];
            s_count[q][threadIdx.x] = run;
            run += c;
        }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kSortRounds; ++r) {
        const long long i = base + r * kSortBlock + threadIdx.x;
        if (i < n) {
            const unsigned d = (key[r] >> shift) & (kDigits - 1);
            const int dst = s_count[r * kWaves + wave][d] + rank[r];
            keys_out[dst] = key[r];
            vals_out[dst] = vals_in ? vals_in[i] : static_cast<int>(i);
        }
    }
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

// ---------------------------------------------------------------- stream form
__global__ void stream_init_kernel(StreamHeader* h, int num_parts, int num_slots, int num_nodes, int generation)
{
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        StreamHeader z = {};
        z.empty_rows = num_nodes;
        z.magic = kPlanMagic;
        z.generation = generation;
        z.num_parts = num_parts;
        z.num_nodes = num_nodes;
        z.num_slots = num_slots;
        *h = z;
    }
}

// is_end[q]: plan entry q is the last of its piece
__global__ __launch_bounds__(256) void stream_ends_kernel(PlanView plan, int num_parts, int* __restrict__ is_end,
                                                         StreamHeader* h)
{
    const int q = blockIdx.x * blockDim.x + threadIdx.x;
    if (q >= num_parts) return;
    const bool nonempty = plan.ptr[q + 1] > plan.ptr[q];
    is_end[q] = nonempty && (plan.flags[q] & 8) == 0;
    if (!nonempty) h->empty_groups = 1;
}

// ends_before[q] = pieces that end before entry q (exclusive scan of is_end; [P] = number of pieces).  Piece e:
// first[e] = its first slot | bit 31 when the row has groups before it, last[e] = its last slot,
// erow[e] = its row | bit 31 when the row has groups after it; the last slot is flagged in col.
__global__ __launch_bounds__(256) void stream_pieces_kernel(PlanView plan, int num_parts,
                                                           const int* __restrict__ ends_before, int* __restrict__ first,
                                                           int* __restrict__ last, int* __restrict__ erow, StreamHeader* h)
{
    const int q = blockIdx.x * blockDim.x + threadIdx.x;
    if (q == 0) h->num_events = ends_before[num_parts];
    if (q >= num_parts) return;
    const int beg = plan.ptr[q], end = plan.ptr[q + 1];
    if (end <= beg) return;
    const int f = plan.flags[q];
    const int e = ends_before[q];
    if (e < 0 || e >= num_parts) return;          // only after a stalled scan (the plan is then refused)
    if ((f & 4) == 0) first[e] = beg | ((f & 1) ? static_cast<int>(kStreamFlag) : 0);
    if ((f & 8) == 0) {
        last[e] = end - 1;
        erow[e] = plan.row[q] | ((f & 2) ? static_cast<int>(kStreamFlag) : 0);
        plan.col[end - 1] |= static_cast<int>(kStreamFlag);
    }
}

// number of pieces whose last slot lies before `slot`
__device__ __forceinline__ int pieces_before(const int* __restrict__ last, int num_events, int slot)
{
    int lo = 0, hi = num_events;
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (last[mid] < slot) lo = mid + 1; else hi = mid;
    }
    return lo;
}

// Candidates for a partial sum: piece e at index e, the tail of wave w at index P + w.  key = the row for a real
// candidate, num_nodes otherwise (sorts behind every row).  Also: plain pieces get their row in erow, every piece
// marks its row as touched, wtail is preset to -1, the padding of col is written.
__global__ __launch_bounds__(256) void stream_classify_kernel(PlanView plan, StreamView sv, int num_parts, int num_slots,
                                                             int padded_slots, int num_nodes,
                                                             const int* __restrict__ first, const int* __restrict__ last,
                                                             unsigned* __restrict__ keys)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    const int num_waves = padded_slots / kStreamWave;
    // "gathers nothing": an id whose row lies behind every table, in swizzled row order too
    if (i < padded_slots - num_slots) plan.col[num_slots + i] = static_cast<int>(swizzle_padded_rows(num_nodes));
    if (i >= num_parts + num_waves) return;
    if (sv.header->empty_groups) { keys[i] = static_cast<unsigned>(num_nodes); if (i >= num_parts) sv.wtail[i - num_parts] = -1; return; }
    const int num_events = sv.header->num_events;
    unsigned key = static_cast<unsigned>(num_nodes);
    if (i < num_parts) {
        if (i < num_events) {
            const int a = first[i], b = last[i], r = sv.erow[i];
            const int row = r & kStreamIdMask;
            const bool whole = a >= 0 && r >= 0;
            const bool partial = !whole || (a & kStreamIdMask) < b / kStreamWave * kStreamWave;
            if (row < num_nodes) atomicOr(sv.touched + (row >> 5), 1u << (row & 31));
            if (partial) key = static_cast<unsigned>(row);
            else sv.erow[i] = row;
        }
    } else {
        const int w = i - num_parts;
        sv.wtail[w] = -1;
        const long long at = static_cast<long long>(w + 1) * kStreamWave - 1;
        if (at < num_slots && plan.col[at] >= 0) {
            const int e = pieces_before(last, num_events, static_cast<int>(at));
            if (e < num_events) key = static_cast<unsigned>(sv.erow[e] & kStreamIdMask);
        }
    }
    keys[i] = key;
}

__global__ __launch_bounds__(256) void stream_cev_kernel(StreamView sv, int num_slots, int padded_slots,
                                                        const int* __restrict__ last)
{
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c > padded_slots / kStreamChunk) return;
    if (sv.header->empty_groups) { sv.cev[c] = 0; return; }
    const int num_events = sv.header->num_events;
    const long long pos = static_cast<long long>(c) * kStreamChunk;
    const int e = pos >= num_slots ? num_events : pieces_before(last, num_events, static_cast<int>(pos));
    const bool inside = pos > 0 && pos < num_slots && !(e > 0 && last[e - 1] == pos - 1);
    sv.cev[c] = e | (inside ? static_cast<int>(kStreamFlag) : 0);
}

// sorted candidates: position k of a real one is the index of its partial sum
__global__ __launch_bounds__(256) void stream_assign_kernel(StreamView sv, int num_parts, int total, int num_nodes,
                                                           const unsigned* __restrict__ sorted_keys,
                                                           const int* __restrict__ order, int* __restrict__ is_head)
{
    const int k = blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= total) return;
    const unsigned key = sorted_keys[k];
    int head = 0;
    if (key < static_cast<unsigned>(num_nodes) && !sv.header->empty_groups) {
        const int src = order[k];
        if (src >= 0 && src < num_parts) sv.erow[src] = static_cast<int>(kStreamFlag) | k;
        else if (src >= num_parts && src < total) sv.wtail[src - num_parts] = k;
        head = k == 0 || sorted_keys[k - 1] != key;
        if (k + 1 == total || sorted_keys[k + 1] >= static_cast<unsigned>(num_nodes)) sv.header->num_partials = k + 1;
    }
    is_head[k] = head;
}

__global__ __launch_bounds__(256) void stream_fix_rows_kernel(StreamView sv, int total, int num_nodes,
                                                             const unsigned* __restrict__ sorted_keys,
                                                             const int* __restrict__ is_head, const int* __restrict__ heads_before)
{
    const int k = blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= total || !is_head[k]) return;
    const int j = heads_before[k];
    if (j < 0 || j >= num_nodes) return;          // only after a stalled scan
    sv.frow[j] = static_cast<int>(sorted_keys[k]);
    sv.fptr[j] = k;
}

__global__ __launch_bounds__(256) void stream_count_rows_kernel(StreamView sv, int words)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    int c = i < words ? __popc(sv.touched[i]) : 0;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) c += __shfl_xor(c, off, kWave);
    if ((threadIdx.x & (kWave - 1)) == 0 && c) atomicSub(&sv.header->empty_rows, c);
}

__global__ void stream_finish_kernel(StreamView sv, const int* __restrict__ heads_before, int total, int num_nodes,
                                     const ScanState* a, const ScanState* b)
{
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    StreamHeader* h = sv.header;
    const int num_fix = h->empty_groups ? 0 : min(max(heads_before[total], 0), num_nodes);
    h->num_fix = num_fix;
    sv.fptr[num_fix] = h->num_partials;
    h->error = (a->error || b->error) ? 1 : 0;
    h->valid = (!h->empty_groups && !h->error) ? 1 : 0;
}

// ---------------------------------------------------------------- host
static size_t scan_state_bytes(long long n)
{
    const long long tiles = (n + kScanTile - 1) / kScanTile;
    return align256(sizeof(ScanState) + sizeof(uint64_t) * static_cast<size_t>(tiles > 0 ? tiles : 1));
}

static long long sort_tiles(long long n) { return (n + kSortTile - 1) / kSortTile; }
// histogram | its exclusive scan (one more entry) | state of that scan
static size_t sort_temp_bytes(long long n)
{
    const long long entries = sort_tiles(n) * kDigits;
    return 2 * align256(sizeof(int) * static_cast<size_t>(entries + 1)) + scan_state_bytes(entries);
}

// The stream form sorts one candidate per plan entry and per wave of the stream kernel.
static long long plan_sort_capacity(long long num_parts, long long num_slots)
{
    return (num_parts > 0 ? num_parts : 0) + stream_padded_slots(num_slots) / kStreamWave;
}

// workspace layout: six arrays of plan_sort_capacity + 1 ints (keys, sorted keys, two index arrays, sizes, one
// more for the stream form) | scan state | sort temporaries
constexpr int kPlanSlabs = 6;
size_t plan_workspace_bytes(long long num_parts, long long num_slots)
{
    if (num_parts <= 0) return 256;
    const long long cap = plan_sort_capacity(num_parts, num_slots);
    return kPlanSlabs * align256(sizeof(int) * (static_cast<size_t>(cap) + 1)) + scan_state_bytes(cap + 1) +
           sort_temp_bytes(cap) + 256;
}

// where launch_build_plan keeps the state of its look-back scans inside the workspace
static size_t plan_scan_state_offset(long long num_parts, long long num_slots)
{
    return kPlanSlabs * align256(sizeof(int) * (static_cast<size_t>(plan_sort_capacity(num_parts, num_slots)) + 1));
}

// ... and the state of the scans inside its radix sorts (one state for all passes; the stall flag survives them)
static size_t plan_sort_state_offset(long long num_parts, long long num_slots)
{
    const long long cap = plan_sort_capacity(num_parts, num_slots);
    const long long entries = sort_tiles(cap) * kDigits;
    return plan_scan_state_offset(num_parts, num_slots) + scan_state_bytes(cap + 1) +
           2 * align256(sizeof(int) * static_cast<size_t>(entries + 1));
}

int workspace_pitch(int dim);   // aggregate.hip

static std::atomic<int> g_force_shift{0};     // process-wide knobs (tuning header), atomics like the ones below
// Plan policy.  Rows of up to 32 * keep slots are kept together instead of being cut at column-block borders, and
// single-group rows may be ordered by length class inside a block.  Negative = chosen per build from the kernel that
// will run over the plan:
//  * stream form (R-MAT 22, ms per epoch of aggregation): rows of up to 32 / 64 / 96 / 128 / 256 slots kept together
//    -> 4.11 / 4.04 / 4.05 / 4.08 / 4.08 without length classes, 4.15 with classes and 256.  Every gather instruction
//    is full whatever the lengths, so the classes only cost locality of the output rows (one-block plan of the
//    last-layer path: 0.227 -> 0.178 ms without them): keep 2, no classes.
//  * group kernel (runs over a plan when the shape is outside the stream kernel's: table of 4 GB or more, rows beyond
//    1024 bytes, stream mode off): equal gather steps per round matter, 256 slots with classes is its optimum and the
//    stream policy costs it 10 % (5.11 against 4.66 ms at R-MAT 22; 22.6 against 20.6 ms at R-MAT 24): keep 8, classes.
static std::atomic<int> g_keep_rows{-1};         // in units of 32 slots
static std::atomic<int> g_length_classes{-1};
void set_plan_length_classes(int on) { g_length_classes.store(on < 0 ? -1 : on ? 1 : 0); }
void set_plan_keep_rows(int keep) { g_keep_rows.store(keep < 0 ? -1 : keep); }
bool stream_covers(int num_nodes, int dim, int ld_in, const float* table);   // stream.hip
static void plan_policy(int num_nodes, int dim, int* keep_rows, int* length_classes)
{
    const bool stream = stream_covers(num_nodes, dim, workspace_pitch(dim), nullptr);
    const int keep = g_keep_rows.load(), classes = g_length_classes.load();
    *keep_rows = keep >= 0 ? keep : stream ? 2 : 8;
    *length_classes = classes >= 0 ? classes : stream ? 0 : 1;
}
void set_schedule_shift(int shift) { g_force_shift.store(shift); }

int schedule_shift(int dim)
{
    if (const int forced = g_force_shift.load(); forced > 0) return forced;
    // column blocks of at most 128K rows and 16 MB of feature rows.  Measured at R-MAT scale 22
    // (ms per epoch, 64- and 128-byte rows): 2^14 5.95, 2^15 5.74, 2^16 5.63, 2^17 5.60, 2^18 5.65,
    // 2^19 5.83 - the window all waves gather from has to stay resident in the memory-side cache,
    // not in one XCD's L2, and larger blocks leave fewer partial sums to combine
    const int row_bytes = 4 * workspace_pitch(dim);
    int shift = 17;
    while (shift > 8 && (static_cast<long long>(row_bytes) << shift) > (16ll << 20)) --shift;
    return shift;
}

// keep_error: a later scan over the same state must not wipe the stall flag of an earlier one
__global__ void plan_scan_init_kernel(ScanState* st, uint64_t* desc, int num_tiles, bool keep_error)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < num_tiles) desc[i] = kTileEmpty;
    if (i == 0) {
        st->counter = 0;
        if (!keep_error) st->error = 0;
        st->counts[0] = st->counts[1] = 0;
        st->overflow = 0;
    }
}

// out[0..n] = exclusive prefix sums of in[0..n) (out[n] = total), with the scan state at `state`
static int launch_exclusive_scan(const int* in, int* out, long long n, void* state, hipStream_t stream,
                                 bool keep_error = false)
{
    ScanState* st = static_cast<ScanState*>(state);
    uint64_t* desc = reinterpret_cast<uint64_t*>(st + 1);
    const int tiles = static_cast<int>((n + kScanTile - 1) / kScanTile);
    hipLaunchKernelGGL(plan_scan_init_kernel, dim3((tiles + 255) / 256), dim3(256), 0, stream, st, desc, tiles, keep_error);
    EPPGCN_HIP(hipGetLastError());
    hipLaunchKernelGGL(exclusive_scan_kernel, dim3(tiles), dim3(kScanBlock), 0, stream, in, out, static_cast<int>(n),
                       tiles, st, desc, scan_mode());
    EPPGCN_HIP(hipGetLastError());
    return kOk;
}

// Sorts the pairs (keys[i], i) by the low `bits` bits of the key, stably; the sorted indices end up in
// `order`.  keys_a is overwritten; keys_b, vals_tmp and temp are scratch.
static int stable_sort_by_key(unsigned* keys_a, unsigned* keys_b, int* vals_tmp, int* order, int n, int bits, void* temp,
                              void* state, hipStream_t stream, unsigned** sorted_keys = nullptr, bool keep_error = false)
{
    const int tiles = static_cast<int>(sort_tiles(n));
    const long long entries = static_cast<long long>(tiles) * kDigits;
    char* t = static_cast<char*>(temp);
    int* hist = reinterpret_cast<int*>(t);
    int* offsets = reinterpret_cast<int*>(t + align256(sizeof(int) * static_cast<size_t>(entries + 1)));
    const int passes = bits <= 8 ? 1 : (bits + 7) / 8;
    // the last pass must write `order`: with an even number of passes the first one writes the temporary
    unsigned* kin = keys_a;
    unsigned* kout = keys_b;
    const int* vin = nullptr;
    for (int pass = 0; pass < passes; ++pass) {
        int* vout = ((passes - pass) % 2 == 1) ? order : vals_tmp;
        const int shift = pass * 8;
        hipLaunchKernelGGL(radix_hist_kernel, dim3(tiles), dim3(kSortBlock), 0, stream, kin, n, shift, tiles, hist);
        EPPGCN_HIP(hipGetLastError());
        if (int rc = launch_exclusive_scan(hist, offsets, entries, state, stream, keep_error || pass > 0)) return rc;
        hipLaunchKernelGGL(radix_scatter_kernel, dim3(tiles), dim3(kSortBlock), 0, stream, kin, vin, kout, vout, n, shift,
                           tiles, offsets);
        EPPGCN_HIP(hipGetLastError());
        unsigned* tk = kin; kin = kout; kout = tk;
        vin = vout;
    }
    if (sorted_keys) *sorted_keys = kin;
    return kOk;
}

static int launch_build_stream(PlanView v, StreamView sv, int num_parts, long long num_slots, int num_nodes, char* base,
                               size_t slab, ScanState* st, ScanState* sort_st, void* temp, int generation,
                               hipStream_t stream)
{
    const int padded = static_cast<int>(stream_padded_slots(num_slots));
    const int num_waves = padded / kStreamWave;
    const int total = num_parts + num_waves;
    int* is_end = reinterpret_cast<int*>(base);                       // later: scratch of the sort
    int* ends_before = reinterpret_cast<int*>(base + slab);           // later: second key array of the sort
    int* first = reinterpret_cast<int*>(base + 2 * slab);             // later: is_head
    int* last = reinterpret_cast<int*>(base + 3 * slab);              // later: heads_before
    unsigned* keys = reinterpret_cast<unsigned*>(base + 4 * slab);
    int* order = reinterpret_cast<int*>(base + 5 * slab);
    const auto blocks = [](long long n) { return dim3(static_cast<unsigned>((n + 255) / 256 > 0 ? (n + 255) / 256 : 1)); };
    hipLaunchKernelGGL(stream_init_kernel, dim3(1), dim3(64), 0, stream, sv.header, num_parts,
                       static_cast<int>(num_slots), num_nodes, generation);
    EPPGCN_HIP(hipGetLastError());
    if (int rc = launch_zero_words(sv.touched, plan_single_words(num_nodes), stream)) return rc;
    hipLaunchKernelGGL(stream_ends_kernel, blocks(num_parts), dim3(256), 0, stream, v, num_parts, is_end, sv.header);
    EPPGCN_HIP(hipGetLastError());
    if (int rc = launch_exclusive_scan(is_end, ends_before, num_parts, st, stream, true)) return rc;
    hipLaunchKernelGGL(stream_pieces_kernel, blocks(num_parts), dim3(256), 0, stream, v, num_parts, ends_before, first, last,
                       sv.erow, sv.header);
    EPPGCN_HIP(hipGetLastError());
    const long long classify_threads = total > padded - num_slots ? total : padded - num_slots;
    hipLaunchKernelGGL(stream_classify_kernel, blocks(classify_threads), dim3(256), 0, stream, v, sv, num_parts,
                       static_cast<int>(num_slots), padded, num_nodes, first, last, keys);
    EPPGCN_HIP(hipGetLastError());
    hipLaunchKernelGGL(stream_cev_kernel, blocks(padded / kStreamChunk + 1), dim3(256), 0, stream, sv,
                       static_cast<int>(num_slots), padded, last);
    EPPGCN_HIP(hipGetLastError());
    int bits = 1;
    while (bits < 31 && (1ll << bits) <= num_nodes) ++bits;           // the key num_nodes needs a digit too
    unsigned* sorted_keys = nullptr;
    if (int rc = stable_sort_by_key(keys, reinterpret_cast<unsigned*>(ends_before), is_end, order, total, bits, temp, sort_st,
                                    stream, &sorted_keys, true))
        return rc;
    int* is_head = first;
    int* heads_before = last;
    hipLaunchKernelGGL(stream_assign_kernel, blocks(total), dim3(256), 0, stream, sv, num_parts, total, num_nodes, sorted_keys,
                       order, is_head);
    EPPGCN_HIP(hipGetLastError());
    if (int rc = launch_exclusive_scan(is_head, heads_before, total, st, stream, true)) return rc;
    hipLaunchKernelGGL(stream_fix_rows_kernel, blocks(total), dim3(256), 0, stream, sv, total, num_nodes, sorted_keys,
                       is_head, heads_before);
    EPPGCN_HIP(hipGetLastError());
    hipLaunchKernelGGL(stream_count_rows_kernel, blocks(static_cast<long long>(plan_single_words(num_nodes))), dim3(256), 0,
                       stream, sv, static_cast<int>(plan_single_words(num_nodes)));
    EPPGCN_HIP(hipGetLastError());
    hipLaunchKernelGGL(stream_finish_kernel, dim3(1), dim3(64), 0, stream, sv, heads_before, total, num_nodes, st,
                       sort_st);
    EPPGCN_HIP(hipGetLastError());
    return kOk;
}

// Every build gets a number of its own (> 0): it is written into the plan's header and remembered by the host with the
// header's counts, so that a kernel can tell the plan it was launched for from other bytes at the same address.
static std::atomic<int> g_plan_generation{0};
static int next_plan_generation()
{
    int g = g_plan_generation.fetch_add(1) + 1;
    if (g <= 0) { g_plan_generation.store(1); g = 1; }      // wrapped after 2^31 builds
    return g;
}
static int last_plan_generation() { return g_plan_generation.load(); }

int launch_build_plan(const int* part_ptr, const int* col, const int* part2node, const int* ids, int num_parts,
                      long long num_slots, int num_nodes, int shift, int dim, void* plan, size_t plan_size,
                      void* workspace, size_t workspace_bytes, hipStream_t stream)
{
    forget_stream_info(plan);
    int keep_rows, length_classes;
    plan_policy(num_nodes, dim, &keep_rows, &length_classes);
    if (num_parts <= 0) return kOk;
    if (plan_size < plan_bytes(num_parts, num_slots, num_nodes)) {
        set_error("build_plan: plan buffer smaller than eppgcn_plan_bytes(num_parts, num_slots, num_nodes)");
        return kErrInvalidArgument;
    }
    if (num_slots >= (1ll << 31) - kStreamWave) {
        set_error("build_plan: slot count beyond 32-bit offsets");
        return kErrInvalidArgument;
    }
    const long long cap = plan_sort_capacity(num_parts, num_slots);
    const size_t slab = align256(sizeof(int) * (static_cast<size_t>(cap) + 1));
    char* base = static_cast<char*>(workspace);
    unsigned* keys_in = reinterpret_cast<unsigned*>(base);
    unsigned* keys_out = reinterpret_cast<unsigned*>(base + slab);
    int* order_tmp = reinterpret_cast<int*>(base + 2 * slab);
    int* order = reinterpret_cast<int*>(base + 3 * slab);
    int* sizes = reinterpret_cast<int*>(base + 4 * slab);
    ScanState* st = reinterpret_cast<ScanState*>(base + plan_scan_state_offset(num_parts, num_slots));
    void* temp = base + kPlanSlabs * slab + scan_state_bytes(cap + 1);
    ScanState* sort_st = reinterpret_cast<ScanState*>(base + plan_sort_state_offset(num_parts, num_slots));
    int bits = 1;
    while (bits < 30 && (static_cast<long long>(num_nodes) >> shift) >= (1ll << bits)) ++bits;
    if (length_classes) bits += 2;
    if (plan_workspace_bytes(num_parts, num_slots) > workspace_bytes) {
        set_error("build_plan: workspace smaller than eppgcn_plan_workspace_bytes(num_parts, num_slots)");
        return kErrInvalidArgument;
    }
    const unsigned blocks = static_cast<unsigned>((num_parts + 255) / 256);
    hipLaunchKernelGGL(plan_keys_kernel, dim3(blocks), dim3(256), 0, stream, part_ptr, col, part2node, ids, num_parts,
                       shift, keep_rows * 32, length_classes, keys_in);
    EPPGCN_HIP(hipGetLastError());
    if (int rc = stable_sort_by_key(keys_in, keys_out, order_tmp, order, num_parts, bits, temp, sort_st, stream)) return rc;
    hipLaunchKernelGGL(plan_sizes_kernel, dim3(blocks), dim3(256), 0, stream, part_ptr, order, num_parts, sizes);
    EPPGCN_HIP(hipGetLastError());
    PlanView v = plan_view(plan, num_parts, num_nodes);
    if (int rc = launch_zero_words(v.single, plan_single_words(num_nodes), stream)) return rc;
    if (int rc = launch_exclusive_scan(sizes, v.ptr, num_parts, st, stream)) return rc;
    const long long threads = static_cast<long long>(num_parts) * 8;
    hipLaunchKernelGGL(plan_fill_kernel, dim3(static_cast<unsigned>((threads + 255) / 256)), dim3(256), 0, stream,
                       part_ptr, col, part2node, ids, order, num_parts, v);
    EPPGCN_HIP(hipGetLastError());
    return launch_build_stream(v, stream_view(plan, num_parts, num_slots, num_nodes), num_parts, num_slots, num_nodes, base,
                               slab, st, sort_st, temp, next_plan_generation(), stream);
}

// ---------------------------------------------------------------- what the host knows about built plans
}  // namespace eppgcn

#include <map>
#include <mutex>

namespace eppgcn {

static std::mutex g_info_mutex;
static std::map<const void*, StreamInfo> g_infos;

const StreamInfo* find_stream_info(const void* plan, StreamInfo* copy)
{
    std::lock_guard<std::mutex> lock(g_info_mutex);
    auto it = g_infos.find(plan);
    if (it == g_infos.end()) return nullptr;
    *copy = it->second;
    return copy;
}
void forget_stream_info(const void* plan)
{
    std::lock_guard<std::mutex> lock(g_info_mutex);
    g_infos.erase(plan);
}
void remember_stream_info(const void* plan, const StreamInfo& info)
{
    std::lock_guard<std::mutex> lock(g_info_mutex);
    g_infos[plan] = info;
}

// Synchronises the stream and reports (once) a header mismatch that a stream or fix-up kernel has seen on the current
// device since the last report.
int read_aggregation_status(hipStream_t stream)
{
    int* words = nullptr;
    if (int rc = plan_fault_address(&words)) return rc;
    int host[kPlanFaultWords] = {0, 0, 0, 0};
    EPPGCN_HIP(hipMemcpyAsync(host, words, sizeof(host), hipMemcpyDeviceToHost, stream));
    EPPGCN_HIP(hipStreamSynchronize(stream));
    if (!host[0]) return kOk;
    if (int rc = launch_zero_words(words, kPlanFaultWords, stream)) return rc;
    set_error(std::string("an aggregation call was given a plan whose header in memory is not the one the library read at "
                          "that address (seen by the ") + (host[1] == 2 ? "fix-up" : "stream") + " kernel: build " +
              std::to_string(host[2]) + " expected, " + std::to_string(host[3]) +
              " found); that call wrote no output.  The plan's memory was overwritten or replaced: rebuild the plan, or "
              "call eppgcn_plan_release when a plan's memory is given up");
    return kErrPlanMismatch;
}

// Synchronises the stream, reads the plan's header and records it; the return code tells whether a look-back scan
// of the build stalled.
int read_plan_status(const void* plan, long long num_parts, long long num_slots, long long num_nodes,
                     long long* partial_rows, hipStream_t stream)
{
    if (partial_rows) *partial_rows = 0;
    if (num_parts <= 0) return kOk;
    StreamInfo info;
    info.num_parts = num_parts; info.num_slots = num_slots; info.num_nodes = num_nodes;
    const StreamView sv = stream_view(const_cast<void*>(plan), num_parts, num_slots, num_nodes);
    EPPGCN_HIP(hipMemcpyAsync(&info.header, sv.header, sizeof(StreamHeader), hipMemcpyDeviceToHost, stream));
    EPPGCN_HIP(hipStreamSynchronize(stream));
    {   // the address of the mismatch mark on this device is looked up here, outside any graph capture
        int* words = nullptr;
        if (int rc = plan_fault_address(&words)) return rc;
    }
    // only a header that a build of this process wrote for these sizes is taken on: its counts size the launches
    const StreamHeader& h = info.header;
    const long long waves = stream_padded_slots(num_slots) / kStreamWave;
    const bool plausible = h.magic == kPlanMagic && h.generation > 0 && h.generation <= last_plan_generation() &&
                           h.num_parts == num_parts && h.num_nodes == num_nodes && h.num_slots == num_slots &&
                           h.num_events >= 0 && h.num_events <= num_parts && h.num_partials >= 0 &&
                           h.num_partials <= num_parts + waves && h.num_fix >= 0 && h.num_fix <= num_nodes &&
                           h.num_fix <= h.num_partials && h.empty_rows >= 0 && h.empty_rows <= num_nodes;
    if (!plausible) {
        forget_stream_info(plan);
        set_error("plan_status: the memory at `plan` does not hold a plan built with these sizes (no build has "
                  "finished there, or its bytes were overwritten); rebuild it with eppgcn_build_plan");
        return kErrPlanMismatch;
    }
    if (info.header.error) {
        forget_stream_info(plan);
        set_error("look-back scan stalled: a tile waited past its spin limit; the plan is invalid");
        return kErrScanStalled;
    }
    remember_stream_info(plan, info);
    if (partial_rows && info.header.valid) *partial_rows = info.header.num_partials;
    return kOk;
}

}  // namespace eppgcn
