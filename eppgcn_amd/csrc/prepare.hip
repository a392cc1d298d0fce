// Execution-path preparation for gfx950 (wave64): path marking from the train
// mask, single-pass stream compaction of the kept edges, splitting of the kept
// edges into backward neighbour groups, forward neighbour groups from the CSR
// row pointers, and the small counting kernels the group-size heuristics need.
//
// Replaces mask_forward_cuda_kernel (EPPGCN/GCNConv/EPPGCN_kernel.cu:351-388), the three
// live cuCompactor namespaces and the thrust scans (EPPGCN/GCNConv/cuCompactor.cu:42-48,
// :328-465, :467-621, :623-680) and the CPU loop of build_part
// (EPPGCN/GCNConv/EPPGCN.cpp:186-227).
//
// Both scans are single-pass "decoupled look-back" scans: a tile publishes its
// aggregate, then its wave 0 walks back over the predecessors' descriptors, 64
// per step, until it meets a tile whose inclusive prefix is known.  Lane ranks
// inside a wave come from a 64-bit ballot and mbcnt; no block-wide bit-sliced
// counting and no second pass over the input.
#include <atomic>
#include <mutex>

#include "common.hpp"

// Scan scratch of the allocation-free compaction entry point: one ScanState and one 64-bit tile
// descriptor per tile of compact_mask_kernel (16384 slots), for inputs of up to 2^30 slots (512 KiB + 32
// bytes per GPU, held until the process ends).  The name is a host-side stand-in; host code only ever uses
// the device address hipGetSymbolAddress returns for it (static_compact_scratch below).
constexpr long long kStaticCompactMaxLength = 1ll << 30;
constexpr long long kStaticCompactTile = 16384;
constexpr size_t kStaticCompactScratchBytes = 32 + 8 * static_cast<size_t>(kStaticCompactMaxLength / kStaticCompactTile);
static __device__ __align__(256) unsigned char scratch[kStaticCompactScratchBytes];

namespace eppgcn {

// ================================================================ scan state init
__global__ void scan_init_kernel(ScanState* st, uint64_t* desc, int num_tiles)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < num_tiles) desc[i] = kTileEmpty;
    if (i == 0) {
        st->counter = 0;
        st->error = 0;
        st->counts[0] = 0;
        st->counts[1] = 0;
        st->overflow = 0;
    }
}

// Test knob for the stall path: with tile 0 muted every look-back runs into its (then tiny) spin limit,
// raises the error flag and carries on, so the kernels still drain and the host sees EPPGCN_ERR_SCAN_STALLED.
static std::atomic<unsigned> g_scan_mode{0};     // process-wide test knob (tuning header)
unsigned scan_mode() { return g_scan_mode.load(); }
void set_scan_test_mode(unsigned spin_limit, int mute_first_tile)
{
    g_scan_mode.store((spin_limit & 0x7fffffffu) | (mute_first_tile ? 0x80000000u : 0u));
}

// ================================================================ path marking
// A wave owns 64 consecutive forward groups (one per lane) and walks the contiguous slot range
// they cover 64 slots at a time, so that the column ids are read and the edge marks written
// with full-width coalesced accesses whatever the group lengths are.  The group (hence the
// row) of a slot is found by a 6-step search over the 64 group starts kept in LDS.  Kept
// slots are counted per group from the wave ballot, the counts of adjacent groups of one row
// are added across lanes, and one atomic per (wave, row) updates node_degs.
constexpr int kMaskBlock = 256;
constexpr int kMaskWaves = kMaskBlock / kWave;

__global__ __launch_bounds__(kMaskBlock) void mask_forward_kernel(
    const int* __restrict__ part2node, const int* __restrict__ part_ptr, const int* __restrict__ col,
    const uint8_t* __restrict__ src_mask, uint8_t* __restrict__ ngh_mask, int* __restrict__ back_edge_mask,
    int* __restrict__ node_degs, int num_parts, int is_last)
{
    __shared__ int s_beg[kMaskWaves][kWave + 1];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const long long g0 = (static_cast<long long>(blockIdx.x) * kMaskWaves + wave) * kWave;
    if (g0 >= num_parts) return;                       // wave-uniform; the LDS rows are wave-private
    const int ng = static_cast<int>(min(static_cast<long long>(kWave), num_parts - g0));

    int beg = 0, end = 0, row = -1;
    bool row_in_src = false;
    if (lane < ng) {
        beg = part_ptr[g0 + lane];
        end = part_ptr[g0 + lane + 1];
        row = part2node[g0 + lane];
        row_in_src = !is_last && end > beg && src_mask[row] != 0;
        if (row_in_src) ngh_mask[row] = 1;
    }
    int* begs = s_beg[wave];
    begs[lane] = lane < ng ? beg : 0x7fffffff;
    if (lane == 0) begs[kWave] = 0x7fffffff;
    __builtin_amdgcn_wave_barrier();
    const int first = __shfl(beg, 0, kWave);
    const int last = __shfl(end, ng - 1, kWave);

    int kept = 0;
    for (int base = first; base < last; base += kWave) {
        const int e = base + lane;
        const bool in_range = e < last;
        int owner = 0;
#pragma unroll
        for (int step = kWave / 2; step > 0; step >>= 1)
            if (begs[owner + step] <= e) owner += step;          // last group starting at or before e
        const int e_row = __shfl(row, owner, kWave);
        const bool e_src = __shfl(static_cast<int>(row_in_src), owner, kWave) != 0;
        bool keep = false;
        if (in_range) {
            const int end_id = col[e];
            keep = src_mask[end_id] != 0;
            if (keep) back_edge_mask[e] = e_row;
            if (e_src) ngh_mask[end_id] = 1;
        }
        const uint64_t ballot = __ballot(keep);
        // this lane's group covers wave slots [lo, hi) of the current 64
        const int lo = min(max(beg - base, 0), kWave);
        const int hi = min(max(end - base, 0), kWave);
        if (hi > lo) {
            const uint64_t below_hi = hi == kWave ? ~0ull : (1ull << hi) - 1ull;
            kept += __popcll(ballot & below_hi & ~((1ull << lo) - 1ull));
        }
    }
    // adjacent lanes whose groups belong to one row form a run: suffix sums within a run, then one
    // atomic per run.  A lane absorbs the lane `off` above only if no run starts in between.
    const int prev_row = __shfl_up(row, 1, kWave);
    const uint64_t heads = __ballot(lane == 0 || prev_row != row);
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const int other = __shfl_down(kept, off, kWave);
        const uint64_t between = (heads >> 1 >> lane) & ((1ull << off) - 1ull);   // lanes lane+1 .. lane+off
        if (lane + off < kWave && between == 0) kept += other;
    }
    if (lane < ng && ((heads >> lane) & 1ull) && kept > 0) atomicAdd(node_degs + row, kept);
}

// ================================================================ compaction
constexpr int kCompactBlock = 256;
constexpr int kCompactItems = 16;
constexpr int kCompactTile = kCompactBlock * kCompactItems;
static_assert(kCompactItems * (kCompactBlock / kWave) == kWave, "one wave scans the per-(slab, wave) counts");

// Tile of the compaction kernel: kCompactMaskItems items per thread, 16384 per tile.  The tile-id counter is one line
// that every workgroup hits with a device-scope atomic, and those serialise; at R-MAT scale 22 (132 M slots) tiles of
// 4096 slots took 0.47 / 0.62 ms (a tenth / nearly all of the slots kept), tiles of 16384 take 0.38 / 0.53 ms.
// 16-byte loads of the mask with the same tile: 0.34 / 0.60 ms (each lane then stores 4 items of its own and a store
// instruction covers every fourth word) - not kept.
constexpr int kCompactMaskItems = 64;
constexpr int kCompactMaskTile = kCompactBlock * kCompactMaskItems;
static_assert(kCompactMaskTile % kCompactTile == 0, "the workspace is sized for tiles of kCompactTile slots");

__global__ __launch_bounds__(kCompactBlock) void compact_mask_kernel(
    const int* __restrict__ in_id, const int* __restrict__ in_edge, int* __restrict__ out_id,
    int* __restrict__ out_edge, int length, int num_tiles, ScanState* st, uint64_t* desc, unsigned mode)
{
    constexpr int kItems = kCompactMaskItems;
    constexpr int kWaves = kCompactBlock / kWave;
    constexpr int kPerLane = kItems * kWaves / kWave;        // counts a lane of the scanning wave adds up
    __shared__ int s_tile;
    __shared__ int s_count[kItems * kWaves];                 // (item k, wave) in output order
    __shared__ int s_prefix;
    const int tile = acquire_tile(st, &s_tile);
    if (tile >= num_tiles) return;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const long long base = static_cast<long long>(tile) * kCompactMaskTile;

    int v[kItems];
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        const long long idx = base + k * kCompactBlock + threadIdx.x;
        v[k] = idx < length ? in_id[idx] : -1;
    }
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        const uint64_t ballot = __ballot(v[k] != -1);
        if (lane == 0) s_count[k * kWaves + wave] = __popcll(ballot);
    }
    __syncthreads();
    if (wave == 0) {
        int c[kPerLane], sum = 0;
#pragma unroll
        for (int j = 0; j < kPerLane; ++j) {
            c[j] = s_count[lane * kPerLane + j];
            sum += c[j];
        }
        const int incl = wave_inclusive_scan(sum);
        const int total = __shfl(incl, kWave - 1, kWave);
        int run = incl - sum;
#pragma unroll
        for (int j = 0; j < kPerLane; ++j) {
            s_count[lane * kPerLane + j] = run;
            run += c[j];
        }
        const uint64_t excl = tile_lookback(desc, st, tile, static_cast<uint64_t>(total), mode);
        if (lane == 0) {
            s_prefix = static_cast<int>(excl);
            if (tile == num_tiles - 1) st->counts[0] = static_cast<int>(excl) + total;
        }
    }
    __syncthreads();
    const int prefix = s_prefix;
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        const bool pred = v[k] != -1;
        const uint64_t ballot = __ballot(pred);
        if (pred) {
            const long long idx = base + k * kCompactBlock + threadIdx.x;
            const int dst = prefix + s_count[k * kWaves + wave] + ballot_rank(ballot);
            out_id[dst] = v[k];
            out_edge[dst] = in_edge[idx];
        }
    }
}

// ================================================================ fused marking + compaction
// One pass over the slots does what mask_forward_kernel followed by compact_mask_kernel do, without
// the E-entry edge mask between them: a tile of 4096 consecutive slots finds the group (hence the
// row) of every slot from a bit map of the group starts inside the tile (prefix population count;
// tile_groups_kernel finds each tile's first group beforehand), decides keep = src_mask[col],
// marks the neighbour masks, counts kept slots per row from wave ballots (one atomic per run of
// equal rows in a wave), and compacts (row, col) of the kept slots with the same ballot ranks and
// look-back prefix as compact_mask_kernel.

// first[t] = last group starting at or before slot t * kCompactTile; first[num_tiles] = last group
__global__ void tile_groups_kernel(const int* __restrict__ part_ptr, int num_parts, int num_tiles,
                                   int* __restrict__ first)
{
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t > num_tiles) return;
    if (t == num_tiles) {
        first[t] = num_parts - 1;
        return;
    }
    const long long slot = static_cast<long long>(t) * kCompactTile;
    int a = 0, b = num_parts;                 // part_ptr[a] <= slot is assumed for a = 0
    while (b - a > 1) {
        const int mid = a + (b - a) / 2;
        if (part_ptr[mid] <= slot) a = mid; else b = mid;
    }
    first[t] = a;
}

__global__ __launch_bounds__(kCompactBlock) void mark_compact_kernel(
    const int* __restrict__ part2node, const int* __restrict__ part_ptr, const int* __restrict__ col,
    const uint8_t* __restrict__ src_mask, uint8_t* __restrict__ ngh_mask, int* __restrict__ node_degs,
    int* __restrict__ out_id, int* __restrict__ out_edge, int num_parts, int length, int num_tiles, int is_last,
    const int* __restrict__ tile_first, ScanState* st, uint64_t* desc, unsigned mode)
{
    __shared__ int s_tile;
    __shared__ int s_count[kWave];
    __shared__ int s_prefix;
    __shared__ unsigned long long s_bits[kCompactTile / 64];   // bit p: a group starts at slot base + p
    __shared__ int s_word_prefix[kCompactTile / 64];     // group starts before each 64-slot word
    __shared__ int s_starts_in_tile;
    if (threadIdx.x < kCompactTile / 64) s_bits[threadIdx.x] = 0ull;
    if (threadIdx.x == 0) s_starts_in_tile = 0;
    const int tile = acquire_tile(st, &s_tile);          // contains the barrier that publishes the zeros
    if (tile >= num_tiles) return;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const long long base = static_cast<long long>(tile) * kCompactTile;
    const int g_lo = tile_first[tile];
    const int g_cnt = tile_first[tile + 1] - g_lo + 1;
    // slots outside [part_ptr[0], part_ptr[num_parts]) belong to no group and are never kept
    const int owned_lo = part_ptr[0];
    const int owned_hi = part_ptr[num_parts];
    // The owner of slot e is g_lo - 1 + (number of groups of the tile that start at or before e).
    // When no two groups start at the same slot (no empty groups, as build_part guarantees) that
    // number is a prefix population count over a 4096-bit map of group starts; otherwise every
    // slot does a binary search over the group starts in global memory.
    {
        int mine = 0;
        for (int i = threadIdx.x; i < g_cnt; i += kCompactBlock) {
            const long long p = part_ptr[g_lo + i] - base;
            if (p >= 0 && p < kCompactTile) {
                atomicOr(&s_bits[p >> 6], 1ull << (p & 63));
                ++mine;
            }
        }
        if (mine) atomicAdd(&s_starts_in_tile, mine);
    }
    __syncthreads();
    if (wave == 0) {
        const int pc = __popcll(s_bits[lane]);
        const int incl = wave_inclusive_scan(pc);
        s_word_prefix[lane] = incl - pc;
        if (lane == kWave - 1 && incl != s_starts_in_tile) s_starts_in_tile = -1;   // duplicate starts
    }
    __syncthreads();
    const bool by_bits = s_starts_in_tile >= 0;
    const int before = part_ptr[g_lo] < base ? 1 : 0;    // g_lo itself starts before the tile

    // phases with all loads of one kind issued together: a ballot inside the item loop would make
    // every item wait for its own gather (16 dependent memory round trips per tile)
    int v[kCompactItems], c[kCompactItems], rows[kCompactItems];
    bool ok[kCompactItems], keep[kCompactItems], row_src[kCompactItems];
#pragma unroll
    for (int k = 0; k < kCompactItems; ++k) {
        const long long idx = base + k * kCompactBlock + threadIdx.x;
        ok[k] = idx < length && idx >= owned_lo && idx < owned_hi;
        c[k] = ok[k] ? col[idx] : 0;
    }
#pragma unroll
    for (int k = 0; k < kCompactItems; ++k) {
        rows[k] = -1;
        if (ok[k]) {
            const int e = static_cast<int>(base + k * kCompactBlock + threadIdx.x);
            int a = 0, b = g_cnt;
            if (by_bits) {
                const int p = k * kCompactBlock + threadIdx.x;
                const unsigned long long upto = (p & 63) == 63 ? ~0ull : (2ull << (p & 63)) - 1ull;
                a = before + s_word_prefix[p >> 6] + __popcll(s_bits[p >> 6] & upto) - 1;
            } else {
                while (b - a > 1) {
                    const int mid = (a + b) >> 1;
                    if (part_ptr[g_lo + mid] <= e) a = mid; else b = mid;
                }
            }
            rows[k] = part2node[g_lo + a];
        }
    }
#pragma unroll
    for (int k = 0; k < kCompactItems; ++k) {
        keep[k] = ok[k] && src_mask[c[k]] != 0;
        row_src[k] = ok[k] && !is_last && src_mask[rows[k]] != 0;
    }
#pragma unroll
    for (int k = 0; k < kCompactItems; ++k) {
        if (row_src[k]) {
            ngh_mask[rows[k]] = 1;
            ngh_mask[c[k]] = 1;
        }
        v[k] = keep[k] ? rows[k] : -1;
        // kept slots per row: the lanes of a wave hold 64 consecutive slots of item k
        const int row = rows[k];
        const int prev_row = __shfl_up(row, 1, kWave);
        const uint64_t heads = __ballot(lane == 0 || prev_row != row);
        const uint64_t kept = __ballot(keep[k]);
        if ((heads >> lane) & 1ull) {
            const uint64_t above = lane == kWave - 1 ? 0ull : heads & ~((2ull << lane) - 1ull);
            const int next = above ? __builtin_ctzll(above) : kWave;
            const uint64_t upto = next == kWave ? ~0ull : (1ull << next) - 1ull;
            const int n = __popcll(kept & upto & ~((1ull << lane) - 1ull));
            if (n > 0) atomicAdd(node_degs + row, n);
        }
        if (lane == 0) s_count[k * (kCompactBlock / kWave) + wave] = __popcll(kept);
    }
    __syncthreads();
    if (wave == 0) {
        const int cnt = s_count[lane];
        const int incl = wave_inclusive_scan(cnt);
        const int total = __shfl(incl, kWave - 1, kWave);
        s_count[lane] = incl - cnt;
        const uint64_t excl = tile_lookback(desc, st, tile, static_cast<uint64_t>(total), mode);
        if (lane == 0) {
            s_prefix = static_cast<int>(excl);
            if (tile == num_tiles - 1) st->counts[0] = static_cast<int>(excl) + total;
        }
    }
    __syncthreads();
    const int prefix = s_prefix;
#pragma unroll
    for (int k = 0; k < kCompactItems; ++k) {
        const bool pred = v[k] != -1;
        const uint64_t ballot = __ballot(pred);
        if (pred) {
            const int dst = prefix + s_count[k * (kCompactBlock / kWave) + wave] + ballot_rank(ballot);
            out_id[dst] = v[k];
            out_edge[dst] = c[k];
        }
    }
}

// Zero both outputs from the compacted length (read on the device) to the end.
__global__ void zero_tail2_kernel(int* __restrict__ a, int* __restrict__ b, const int* __restrict__ d_start, int length)
{
    const long long start = *d_start;
    const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
    for (long long i = start + static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; i < length; i += stride) {
        a[i] = 0;
        b[i] = 0;
    }
}

__global__ void zero_tail1_kernel(int* __restrict__ a, const int* __restrict__ d_start, int offset, long long length)
{
    const long long start = static_cast<long long>(*d_start) + offset;
    const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
    for (long long i = start + static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; i < length; i += stride)
        a[i] = 0;
}

// ================================================================ counting
__global__ __launch_bounds__(256) void count_nonzero_kernel(const int* __restrict__ in, int length, int* __restrict__ d_count)
{
    int local = 0;
    const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
    for (long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; i < length; i += stride)
        local += in[i] != 0;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) local += __shfl_xor(local, off, kWave);
    if ((threadIdx.x & (kWave - 1)) == 0 && local) atomicAdd(d_count, local);
}

// bitmap bit c is set for every c = list[i], i < length; *d_count receives the number of distinct values.
// A bit that already reads as set is not touched again, so the atomics are about one per distinct value
// and wave, not one per entry.
__global__ __launch_bounds__(256) void mark_listed_rows_kernel(const int* __restrict__ list, long long length,
                                                               uint32_t* __restrict__ bitmap, int* __restrict__ d_count)
{
    int fresh = 0;
    const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
    for (long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; i < length; i += stride) {
        const unsigned c = static_cast<unsigned>(list[i]);
        const uint32_t bit = 1u << (c & 31);
        if ((bitmap[c >> 5] & bit) == 0)
            fresh += (atomicOr(bitmap + (c >> 5), bit) & bit) == 0;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) fresh += __shfl_xor(fresh, off, kWave);
    if ((threadIdx.x & (kWave - 1)) == 0 && fresh) atomicAdd(d_count, fresh);
}

// Degree histogram of get_ginfo (EPPGCN/GCNConv/EPPGCN.cpp:356-377): hist[0] = #(deg != 0),
// hist[3..9] = the seven buckets, the last one also taking deg <= 0 and deg >= 160.
__global__ __launch_bounds__(256) void ginfo_hist_kernel(const int* __restrict__ node_deg, int length, int* __restrict__ hist)
{
    int local[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
    for (long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; i < length; i += stride) {
        const int deg = node_deg[i];
        local[0] += deg != 0;
        int b = 7;
        if (deg >= 1 && deg < 5) b = 1;
        else if (deg >= 5 && deg < 10) b = 2;
        else if (deg >= 10 && deg < 20) b = 3;
        else if (deg >= 20 && deg < 40) b = 4;
        else if (deg >= 40 && deg < 80) b = 5;
        else if (deg >= 80 && deg < 160) b = 6;
#pragma unroll
        for (int k = 1; k < 8; ++k) local[k] += b == k;
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        int s = local[k];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, kWave);
        if ((threadIdx.x & (kWave - 1)) == 0 && s) atomicAdd(hist + (k == 0 ? 0 : k + 2), s);
    }
}

// ================================================================ group splitting
// Vertex i with g_i slots (g_i = kept degree, or CSR degree) yields q_i = ceil(g_i/ps)
// groups; group j of vertex i starts at G_i + j*ps where G_i is the exclusive sum
// of g.  One look-back scan carries (sum q, sum g) packed as q*2^31 + g.  The
// tile's groups are then written in two ways: a vertex with at most kSmallGroups
// groups by the thread that owns it, every other vertex - collected on a list in
// LDS - by a whole wave, 64 groups per step with coalesced stores, so a hub vertex
// with a hundred thousand groups costs its tile a longer loop, not one thread a
// longer life.
constexpr int kSplitBlock = 256;
constexpr int kSplitItems = 8;
constexpr int kSplitTile = kSplitBlock * kSplitItems;
constexpr int kSmallGroups = 4;     // groups per vertex up to which the owning thread writes them itself

template <bool kFromRowPtr>
__global__ __launch_bounds__(kSplitBlock) void split_groups_kernel(
    const int* __restrict__ src, int num_nodes, int part_size, int* __restrict__ part_ptr_out,
    int* __restrict__ part2node_out, long long capacity, int num_tiles, ScanState* st, uint64_t* desc, unsigned mode)
{
    __shared__ int s_tile;
    __shared__ int s_q[kSplitTile + 1];
    __shared__ int s_g[kSplitTile];
    __shared__ uint64_t s_wave[kSplitBlock / kWave];
    __shared__ uint64_t s_tile_excl;
    __shared__ int s_big[kSplitTile];
    __shared__ int s_big_count;
    const int tile = acquire_tile(st, &s_tile);
    if (tile >= num_tiles) return;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const long long base = static_cast<long long>(tile) * kSplitTile;

    int g[kSplitItems], q[kSplitItems];
    int tq = 0, tg = 0;
#pragma unroll
    for (int j = 0; j < kSplitItems; ++j) {
        const long long i = base + threadIdx.x * kSplitItems + j;
        int gi = 0;
        if (i < num_nodes) gi = kFromRowPtr ? src[i + 1] - src[i] : src[i];
        gi = gi > 0 ? gi : 0;
        g[j] = gi;
        q[j] = (gi + part_size - 1) / part_size;
        tq += q[j];
        tg += gi;
    }
    const uint64_t mine = (static_cast<uint64_t>(tq) << 31) | static_cast<uint64_t>(tg);
    const uint64_t incl = wave_inclusive_scan_u64(mine);
    if (lane == kWave - 1) s_wave[wave] = incl;
    __syncthreads();
    uint64_t wave_excl = 0, tile_total = 0;
#pragma unroll
    for (int w = 0; w < kSplitBlock / kWave; ++w) {
        if (w < wave) wave_excl += s_wave[w];
        tile_total += s_wave[w];
    }
    if (wave == 0) {
        const uint64_t excl = tile_lookback(desc, st, tile, tile_total, mode);
        if (lane == 0) s_tile_excl = excl;
    }
    // tile-relative q offsets and absolute g offsets of this thread's vertices
    uint64_t run = wave_excl + incl - mine;
    const int g_first = kFromRowPtr ? src[0] : 0;
    __syncthreads();
    const uint64_t tile_excl = s_tile_excl;
    const int q_base = static_cast<int>(tile_excl >> 31);
    const int g_base = static_cast<int>(tile_excl & 0x7fffffffull) + g_first;
#pragma unroll
    for (int j = 0; j < kSplitItems; ++j) {
        const int slot = threadIdx.x * kSplitItems + j;
        s_q[slot] = static_cast<int>(run >> 31);
        s_g[slot] = g_base + static_cast<int>(run & 0x7fffffffull);
        run += (static_cast<uint64_t>(q[j]) << 31) | static_cast<uint64_t>(g[j]);
    }
    const int tile_q = static_cast<int>(tile_total >> 31);
    if (threadIdx.x == 0) {
        s_q[kSplitTile] = tile_q;
        s_big_count = 0;
    }
    __syncthreads();

    // A vertex with at most kSmallGroups groups is written by the thread that owns it; the others
    // go on a list and are written by whole waves, 64 groups per step, so that a tile full of hubs
    // (the first vertices of an R-MAT graph have 10^5 groups each) costs coalesced stores only.
#pragma unroll
    for (int j = 0; j < kSplitItems; ++j) {
        const int slot = threadIdx.x * kSplitItems + j;
        if (q[j] > kSmallGroups) {
            s_big[atomicAdd(&s_big_count, 1)] = slot;
        } else {
            const int start = s_g[slot];
            const long long first = static_cast<long long>(q_base) + s_q[slot];
            for (int k = 0; k < q[j]; ++k) {
                const long long dst = first + k;
                if (dst < capacity) {
                    part_ptr_out[dst] = start + k * part_size;
                    if (part2node_out && dst + 1 < capacity) part2node_out[dst] = static_cast<int>(base) + slot;
                }
            }
        }
    }
    __syncthreads();
    const int big = s_big_count;
    for (int b = wave; b < big; b += kSplitBlock / kWave) {
        const int slot = s_big[b];
        const int count = s_q[slot + 1] - s_q[slot];
        const int start = s_g[slot];
        const long long first = static_cast<long long>(q_base) + s_q[slot];
        for (int k = lane; k < count; k += kWave) {
            const long long dst = first + k;
            if (dst < capacity) {
                part_ptr_out[dst] = start + k * part_size;
                if (part2node_out && dst + 1 < capacity) part2node_out[dst] = static_cast<int>(base) + slot;
            }
        }
    }
    if (tile == num_tiles - 1 && threadIdx.x == 0) {
        const uint64_t total = tile_excl + tile_total;
        const int total_q = static_cast<int>(total >> 31);
        const int total_g = static_cast<int>(total & 0x7fffffffull);
        st->counts[0] = total_q;
        st->counts[1] = total_g;
        if (total_q < capacity) part_ptr_out[total_q] = total_g + g_first;
        if (static_cast<long long>(total_q) + 1 > capacity) st->overflow = 1;
    }
}

// ================================================================ host launchers
__global__ __launch_bounds__(256) void zero_words_kernel(uint32_t* __restrict__ p, size_t head, size_t vecs, size_t words)
{
    // [0, head) scalar words up to the first 16-byte boundary, then `vecs` uint4, then the rest
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    const size_t tid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    uint4* v = reinterpret_cast<uint4*>(p + head);
    // non-temporal: the zeros are not read back before the kernel that follows has filled the caches
    typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
    const uintx4 zero = {0u, 0u, 0u, 0u};
    for (size_t i = tid; i < vecs; i += stride) __builtin_nontemporal_store(zero, reinterpret_cast<uintx4*>(v) + i);
    const size_t tail = head + 4 * vecs;
    if (tid < head) p[tid] = 0u;
    if (tid < words - tail) p[tail + tid] = 0u;
}

int launch_zero_words(void* p, size_t words, hipStream_t stream)
{
    if (words == 0) return kOk;
    const uintptr_t a = reinterpret_cast<uintptr_t>(p);
    size_t head = ((16 - a % 16) % 16) / 4;
    if (head > words) head = words;
    const size_t vecs = (words - head) / 4;
    size_t blocks = (vecs + 255) / 256;
    if (blocks > 256 * 64) blocks = 256 * 64;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(zero_words_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream,
                       static_cast<uint32_t*>(p), head, vecs, words);
    EPPGCN_HIP(hipGetLastError());
    return kOk;
}

// out[num_rows, dim]: one thread per vector of VW floats; a row whose bit in `skip` is set is left alone.
// Index: unsigned when the vector count fits in 32 bits (the row of a vector is then a 32-bit division).
template <int VW, class Index>
__global__ __launch_bounds__(256) void zero_rows_unless_kernel(float* __restrict__ out, const uint32_t* __restrict__ skip,
                                                               Index total_vecs, Index vecs_per_row)
{
    typedef float fvec __attribute__((ext_vector_type(VW)));
    const Index stride = static_cast<Index>(gridDim.x) * blockDim.x;
    for (Index i = static_cast<Index>(blockIdx.x) * blockDim.x + threadIdx.x; i < total_vecs; i += stride) {
        const Index r = i / vecs_per_row;
        if (!((skip[r >> 5] >> (r & 31)) & 1u)) {
            if constexpr (VW == 1) {
                __builtin_nontemporal_store(0.f, out + i);
            } else {
                fvec z = {};
                __builtin_nontemporal_store(z, reinterpret_cast<fvec*>(out) + i);
            }
        }
        if (total_vecs - i <= stride) break;      // the next index would run past the end (and could wrap)
    }
}

// The same with the work found by whole waves: a wave looks at 64 rows at a time, collects those whose bit
// is clear (usually few: the rows of several groups or of none) and clears them VW floats per lane, so
// the cost follows the rows that are cleared instead of the size of the matrix.
template <int VW>
__global__ __launch_bounds__(256) void zero_listed_rows_kernel(float* __restrict__ out, const uint32_t* __restrict__ skip,
                                                               unsigned num_rows, unsigned vecs_per_row)
{
    typedef float fvec __attribute__((ext_vector_type(VW)));
    __shared__ int lists[4][kWave];
    int* list = lists[threadIdx.x / kWave];
    const unsigned lane = lane_id();
    const unsigned waves = gridDim.x * 4u;
    const unsigned blocks64 = (num_rows + 63u) / 64u;
    for (unsigned b = blockIdx.x * 4u + threadIdx.x / kWave; b < blocks64; b += waves) {
        const unsigned r = b * 64u + lane;
        const bool wanted = r < num_rows && ((skip[r >> 5] >> (r & 31)) & 1u) == 0;
        const unsigned count = compact_wanted_rows(list, r, wanted);
        const unsigned total = count * vecs_per_row;
        for (unsigned t = lane; t < total; t += kWave) {
            const unsigned k = t / vecs_per_row;
            const size_t at = static_cast<size_t>(list[k]) * vecs_per_row + (t - k * vecs_per_row);
            if constexpr (VW == 1) {
                __builtin_nontemporal_store(0.f, out + at);
            } else {
                fvec z = {};
                __builtin_nontemporal_store(z, reinterpret_cast<fvec*>(out) + at);
            }
        }
    }
}

static std::atomic<bool> g_force_wide_index{false};
bool force_wide_index() { return g_force_wide_index.load(); }
void set_force_wide_index(bool on) { g_force_wide_index.store(on); }

int launch_zero_rows_unless(float* out, const uint32_t* skip, long long num_rows, int dim, hipStream_t stream)
{
    if (num_rows <= 0 || dim <= 0) return kOk;
    const uintptr_t a = reinterpret_cast<uintptr_t>(out);
    const int vw = (dim % 4 == 0 && a % 16 == 0) ? 4 : (dim % 2 == 0 && a % 8 == 0) ? 2 : 1;
    const int vecs_per_row = dim / vw;
    if (num_rows < (1ll << 31) && !force_wide_index()) {
        long long blocks = (num_rows + 255) / 256;           // one wave per 64 rows
        if (blocks > 256 * 16) blocks = 256 * 16;
        const dim3 grid(static_cast<unsigned>(blocks)), block(256);
        const unsigned n = static_cast<unsigned>(num_rows), v = static_cast<unsigned>(vecs_per_row);
        if (vw == 4) hipLaunchKernelGGL(zero_listed_rows_kernel<4>, grid, block, 0, stream, out, skip, n, v);
        else if (vw == 2) hipLaunchKernelGGL(zero_listed_rows_kernel<2>, grid, block, 0, stream, out, skip, n, v);
        else hipLaunchKernelGGL(zero_listed_rows_kernel<1>, grid, block, 0, stream, out, skip, n, v);
    } else {
        // any size: one thread per vector of the matrix
        const unsigned long long total = static_cast<unsigned long long>(num_rows) * vecs_per_row;
        unsigned long long blocks = (total + 255) / 256;
        if (blocks > 256 * 64) blocks = 256 * 64;
        const dim3 grid(static_cast<unsigned>(blocks)), block(256);
        const unsigned long long v = static_cast<unsigned long long>(vecs_per_row);
        if (vw == 4) hipLaunchKernelGGL((zero_rows_unless_kernel<4, unsigned long long>), grid, block, 0, stream, out, skip, total, v);
        else if (vw == 2) hipLaunchKernelGGL((zero_rows_unless_kernel<2, unsigned long long>), grid, block, 0, stream, out, skip, total, v);
        else hipLaunchKernelGGL((zero_rows_unless_kernel<1, unsigned long long>), grid, block, 0, stream, out, skip, total, v);
    }
    EPPGCN_HIP(hipGetLastError());
    return kOk;
}

size_t scan_workspace_bytes(long long length, int tile)
{
    const long long tiles = (length + tile - 1) / tile;
    return sizeof(ScanState) + sizeof(uint64_t) * static_cast<size_t>(tiles > 0 ? tiles : 1);
}

size_t compact_workspace_bytes(long long length) { return scan_workspace_bytes(length, kCompactTile); }
size_t split_workspace_bytes(long long num_nodes) { return scan_workspace_bytes(num_nodes, kSplitTile); }

static int init_scan(void* workspace, int num_tiles, hipStream_t stream)
{
    ScanState* st = static_cast<ScanState*>(workspace);
    uint64_t* desc = reinterpret_cast<uint64_t*>(st + 1);
    const int n = num_tiles > 0 ? num_tiles : 1;
    hipLaunchKernelGGL(scan_init_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, st, desc, num_tiles);
    EPPGCN_HIP(hipGetLastError());
    return kOk;
}

int launch_mask_forward(const int* part2node, const int* part_ptr, const int* col, const uint8_t* src_mask,
                        uint8_t* ngh_mask, int* back_edge_mask, int* node_degs, int num_parts,
                        long long num_edges, int is_last, hipStream_t stream)
{
    (void)num_edges;
    if (num_parts == 0) return kOk;
    const long long groups_per_block = static_cast<long long>(kWave) * kMaskWaves;
    const unsigned grid = static_cast<unsigned>((num_parts + groups_per_block - 1) / groups_per_block);
    hipLaunchKernelGGL(mask_forward_kernel, dim3(grid), dim3(kMaskBlock), 0, stream, part2node, part_ptr, col, src_mask,
                       ngh_mask, back_edge_mask, node_degs, num_parts, is_last);
    EPPGCN_HIP(hipGetLastError());
    return kOk;
}

// Results land in the ScanState at the head of the workspace: counts[0] = kept length.
int launch_compact_mask(const int* in_id, int* out_id, const int* in_edge, int* out_edge, long long length,
                        void* workspace, hipStream_t stream)
{
    ScanState* st = static_cast<ScanState*>(workspace);
    uint64_t* desc = reinterpret_cast<uint64_t*>(st + 1);
    const int num_tiles = static_cast<int>((length + kCompactMaskTile - 1) / kCompactMaskTile);
    if (int rc = init_scan(workspace, num_tiles, stream)) return rc;
    if (num_tiles > 0) {
        hipLaunchKernelGGL(compact_mask_kernel, dim3(num_tiles), dim3(kCompactBlock), 0, stream, in_id, in_edge,
                           out_id, out_edge, static_cast<int>(length), num_tiles, st, desc, scan_mode());
        EPPGCN_HIP(hipGetLastError());
        long long blocks = (length + 1023) / 1024;
        if (blocks > 2048) blocks = 2048;
        hipLaunchKernelGGL(zero_tail2_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, out_id,
                           out_edge, st->counts, static_cast<int>(length));
        EPPGCN_HIP(hipGetLastError());
    }
    return kOk;
}

// ---- allocation-free compaction: the scan workspace is the file-scope device array `scratch`
long long static_compact_max_length() { return kStaticCompactMaxLength; }

// Device address of `scratch` on the current device, looked up once per device (every GPU holds
// its own copy of the array at its own address).
static int static_compact_scratch(void** out)
{
    constexpr int kMaxDevices = 64;
    static std::mutex lock;
    static void* address[kMaxDevices] = {nullptr};
    int device = 0;
    EPPGCN_HIP(hipGetDevice(&device));
    if (device < 0 || device >= kMaxDevices) {
        set_error("static scratch: device ordinal " + std::to_string(device) + " is outside 0..63");
        return kErrInvalidArgument;
    }
    std::lock_guard<std::mutex> guard(lock);
    if (!address[device]) {
        void* p = nullptr;
        EPPGCN_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p || reinterpret_cast<uintptr_t>(p) % 8 != 0) {
            set_error("static scratch: hipGetSymbolAddress returned an unusable address");
            return kErrHip;
        }
        address[device] = p;
    }
    *out = address[device];
    return kOk;
}

// The scratch address for the status call (and the look-up of the address outside a graph capture).
int static_compact_workspace(void** out) { return static_compact_scratch(out); }

// compact_mask_kernel over the static scratch; *workspace_out receives the scratch address (its
// ScanState holds the kept length once the stream has run).  The scan state and the descriptors of
// the tiles this call uses are cleared by init_scan's fill kernel on every call: the array keeps
// the previous call's contents.
int launch_compact_mask_static(const int* in_id, int* out_id, const int* in_edge, int* out_edge, long long length,
                               void** workspace_out, hipStream_t stream)
{
    static_assert(kStaticCompactTile == kCompactMaskTile && kStaticCompactMaxLength % kCompactMaskTile == 0 &&
                      kStaticCompactScratchBytes == sizeof(ScanState) + 8 * (kStaticCompactMaxLength / kCompactMaskTile),
                  "the static scratch holds the scan state and one descriptor per tile of compact_mask_kernel");
    void* ws = nullptr;
    if (int rc = static_compact_scratch(&ws)) return rc;
    *workspace_out = ws;
    return launch_compact_mask(in_id, out_id, in_edge, out_edge, length, ws, stream);
}

size_t mark_compact_workspace_bytes(long long length)
{
    const long long tiles = (length + kCompactTile - 1) / kCompactTile;
    return compact_workspace_bytes(length) + static_cast<size_t>(tiles + 2) * sizeof(int);
}

// Results land in the ScanState at the head of the workspace: counts[0] = kept length.
int launch_mark_compact(const int* part2node, const int* part_ptr, const int* col, const uint8_t* src_mask,
                        uint8_t* ngh_mask, int* node_degs, int* out_id, int* out_edge, int num_parts,
                        long long length, int is_last, void* workspace, hipStream_t stream)
{
    ScanState* st = static_cast<ScanState*>(workspace);
    uint64_t* desc = reinterpret_cast<uint64_t*>(st + 1);
    const int num_tiles = num_parts > 0 ? static_cast<int>((length + kCompactTile - 1) / kCompactTile) : 0;
    if (int rc = init_scan(workspace, num_tiles, stream)) return rc;
    if (num_tiles == 0) {
        if (length > 0) {
            if (int rc = launch_zero_words(out_id, static_cast<size_t>(length), stream)) return rc;
            if (int rc = launch_zero_words(out_edge, static_cast<size_t>(length), stream)) return rc;
        }
        return kOk;
    }
    int* tile_first = reinterpret_cast<int*>(static_cast<char*>(workspace) + compact_workspace_bytes(length));
    hipLaunchKernelGGL(tile_groups_kernel, dim3((num_tiles + 1 + 255) / 256), dim3(256), 0, stream, part_ptr, num_parts,
                       num_tiles, tile_first);
    EPPGCN_HIP(hipGetLastError());
    hipLaunchKernelGGL(mark_compact_kernel, dim3(num_tiles), dim3(kCompactBlock), 0, stream, part2node, part_ptr, col,
                       src_mask, ngh_mask, node_degs, out_id, out_edge, num_parts, static_cast<int>(length), num_tiles,
                       is_last, tile_first, st, desc, scan_mode());
    EPPGCN_HIP(hipGetLastError());
    long long blocks = (length + 1023) / 1024;
    if (blocks > 2048) blocks = 2048;
    hipLaunchKernelGGL(zero_tail2_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, out_id, out_edge,
                       st->counts, static_cast<int>(length));
    EPPGCN_HIP(hipGetLastError());
    return kOk;
}

// counts[0] = number of groups, counts[1] = number of slots covered.
int launch_split(bool from_row_ptr, const int* src, int num_nodes, int part_size, int* part_ptr_out,
                 int* part2node_out, long long capacity, bool zero_tail, void* workspace, hipStream_t stream)
{
    ScanState* st = static_cast<ScanState*>(workspace);
    uint64_t* desc = reinterpret_cast<uint64_t*>(st + 1);
    const int num_tiles = (num_nodes + kSplitTile - 1) / kSplitTile;
    if (int rc = init_scan(workspace, num_tiles, stream)) return rc;
    if (num_tiles == 0) {
        if (capacity > 0)
            if (int rc = launch_zero_words(part_ptr_out, static_cast<size_t>(zero_tail ? capacity : 1), stream)) return rc;
        return kOk;
    }
    if (from_row_ptr)
        hipLaunchKernelGGL((split_groups_kernel<true>), dim3(num_tiles), dim3(kSplitBlock), 0, stream, src, num_nodes,
                           part_size, part_ptr_out, part2node_out, capacity, num_tiles, st, desc, scan_mode());
    else
        hipLaunchKernelGGL((split_groups_kernel<false>), dim3(num_tiles), dim3(kSplitBlock), 0, stream, src, num_nodes,
                           part_size, part_ptr_out, part2node_out, capacity, num_tiles, st, desc, scan_mode());
    EPPGCN_HIP(hipGetLastError());
    if (zero_tail) {
        long long blocks = (capacity + 1023) / 1024;
        if (blocks > 2048) blocks = 2048;
        if (blocks < 1) blocks = 1;
        hipLaunchKernelGGL(zero_tail1_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, part_ptr_out,
                           st->counts, 1, capacity);
        EPPGCN_HIP(hipGetLastError());
    }
    return kOk;
}

int launch_count_nonzero(const int* in, long long length, int* d_count, hipStream_t stream)
{
    if (int rc = launch_zero_words(d_count, 1, stream)) return rc;
    if (length == 0) return kOk;
    long long blocks = (length + 1023) / 1024;
    if (blocks > 1024) blocks = 1024;
    hipLaunchKernelGGL(count_nonzero_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, in,
                       static_cast<int>(length), d_count);
    EPPGCN_HIP(hipGetLastError());
    return kOk;
}

int launch_mark_listed_rows(const int* list, long long length, long long num_rows, uint32_t* bitmap, int* d_count,
                            hipStream_t stream)
{
    if (int rc = launch_zero_words(bitmap, static_cast<size_t>((num_rows + 31) / 32), stream)) return rc;
    if (int rc = launch_zero_words(d_count, 1, stream)) return rc;
    if (length == 0) return kOk;
    long long blocks = (length + 1023) / 1024;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(mark_listed_rows_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, list, length,
                       bitmap, d_count);
    EPPGCN_HIP(hipGetLastError());
    return kOk;
}

int launch_ginfo_hist(const int* node_deg, long long length, int* d_hist10, hipStream_t stream)
{
    if (int rc = launch_zero_words(d_hist10, 10, stream)) return rc;
    if (length == 0) return kOk;
    long long blocks = (length + 1023) / 1024;
    if (blocks > 1024) blocks = 1024;
    hipLaunchKernelGGL(ginfo_hist_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, node_deg,
                       static_cast<int>(length), d_hist10);
    EPPGCN_HIP(hipGetLastError());
    return kOk;
}

}  // namespace eppgcn
