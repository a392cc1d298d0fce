// Slot-stream aggregation for gfx950 (wave64): the aggregation of a planned launch as a segmented sum
// over one stream of slots, every wave taking the same number of slots.
//
// Same contract as aggregate_kernel (EPPGCN/GCNConv/EPPGCN_kernel.cu:204-295, :626-670):
//
//   out[r, :] = s[r] * sum over the slots e of row r of  table[col[e], :]       (table[c, :] = s[c] * in[c, :])
//
// A plan lists the groups in processing order; consecutive groups that continue one another form a
// "piece" (a stretch of slots of one row).  The stream form of the plan (schedule.hip) is
//
//   scol[S_pad]   column id of every slot in processing order; bit 31 set on the last slot of a piece;
//                 padded to a multiple of kStreamWave slots with an id behind the table ("gathers nothing")
//   erow[NE]      one entry per piece, in stream order: its row when one store writes it (the piece is all of
//                 its row and lies inside one wave's slots), else bit 31 | the index of its partial sum
//   cev[S_pad / 32 + 1]   number of pieces that end before slot 32 c; bit 31 set when slot 32 c lies inside
//                 a piece that started earlier
//   wtail[S_pad / 512]    index of the partial sum of what wave w holds after its last slot, or -1
//   frow, fptr    the rows that have partial sums and the range of each (numbered row by row)
//
// Mapping.  A wave takes kStreamWave = 512 consecutive slots with two 16-byte loads per lane: lane l
// holds slots 8l .. 8l+7.  A team of TS lanes (TS * 16 bytes = one table row) owns the 8 * TS slots its
// own lanes hold and walks them in TS steps of 8 row gathers; the ids of step s are broadcast from lane
// s of the team, so no id goes through LDS or is loaded twice.  Every gather instruction of the wave is
// full (64 / TS rows) whatever the lengths of the rows.  A team adds rows into its partial sum and, at a
// slot that ends a piece, writes the sum to that piece's row (s[r] and r come from a per-wave list in LDS,
// staged once with coalesced loads).  What a team holds at the ends of its slot range - the tail of a piece
// that goes on in the next team, the head of one that began in an earlier team - is combined across the
// teams of the wave once, at the end, with a segmented scan in registers.  Pieces that cross waves and rows cut
// into several pieces leave unscaled partial sums in a scratch area, which a second small kernel adds up row by
// row in a fixed order: no float atomics, no output clear for rows that have slots, and the same bits every run.
#include <type_traits>

#include "common.hpp"

namespace eppgcn {

constexpr int kStreamBlock = 256;
constexpr int kStreamWaves = kStreamBlock / kWave;
constexpr int kStreamShiftTeams = 8;   // teams up to this size address rows with a shift (power-of-two row pitch)
constexpr int kStreamEvents = kStreamWave;       // pieces that can end in a wave's slots
constexpr unsigned kNoRowOffset = 0xffffffffu;

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// How a team writes the floats of an output row it owns (lane tl holds columns 4 tl .. 4 tl + 3):
//   kStoreExact  the row is exactly the team's TS * 16 bytes and 16-byte aligned (widths 16, 32, 64, ...): every lane
//                stores its 16 bytes, non-temporally, and a partial sum (one table row wide) is stored the same way
//   kStoreVec4   the width is a multiple of 4 floats, rows 16-byte aligned: the lanes below the width store 16 bytes,
//                non-temporally (whole 16-byte units written once and never read here)
//   kStorePlain  any width and alignment: 16 bytes per lane while four columns are left, then 8 and 4.  Such rows share
//                their 32-byte sectors with their neighbours, which other teams write at other times: plain stores let
//                the cache put a sector together before it goes to memory (width 22, 88-byte rows at R-MAT 22: forward
//                call 1.589 -> 1.566 ms with plain instead of non-temporal stores; for 64-byte rows the other way round:
//                1.092 -> 1.137 ms).  The pieces are only as aligned as the rows (4 or 8 bytes), which vector memory
//                accesses of whole dwords may be.
enum : int { kStoreExact = 0, kStoreVec4 = 1, kStorePlain = 2 };
typedef float f32x4u __attribute__((ext_vector_type(4), aligned(4)));
typedef float f32x2u __attribute__((ext_vector_type(2), aligned(4)));

template <int MODE>
__device__ __forceinline__ void store_row_floats(float* p, const float (&v)[4], int n)
{
    if constexpr (MODE != kStorePlain) {
        if (MODE == kStoreExact || n > 0) {
            const f32x4 t = {v[0], v[1], v[2], v[3]};
            __builtin_nontemporal_store(t, reinterpret_cast<f32x4*>(p));
        }
    } else {
        if (n >= 4) {
            *reinterpret_cast<f32x4u*>(p) = f32x4u{v[0], v[1], v[2], v[3]};
        } else if (n > 0) {
            if (n & 2) *reinterpret_cast<f32x2u*>(p) = f32x2u{v[0], v[1]};
            if (n & 1) p[n & 2] = v[n & 2];
        }
    }
}

// table rows: pitch ld_bytes (a multiple of 16), `chunks` 16-byte vectors of a row are read (chunks <= TS);
// out rows: pitch ld_out floats, columns < width_out written as the store mode says;
// partial rows: pitch ld_bytes, written whole (unscaled sums).
// U: row gathers per batch (4 or 8); two batches are in flight.
template <int U> struct StreamBatch {
    u32x4 v[U];
    unsigned c[U];
};

// Is the header in memory the one the host remembers for this plan address?  (num_events < 0: not compared)
__device__ __forceinline__ bool header_mismatch(const StreamHeader* __restrict__ h, int generation, int num_events,
                                                int num_partials)
{
    return h->valid != 1 || h->magic != kPlanMagic || h->generation != generation || h->num_partials != num_partials ||
           (num_events >= 0 && h->num_events != num_events);
}
// One lane leaves the mark in the library's own device words (ordinary vector stores; the plan's memory is not
// written: whatever replaced the plan there belongs to somebody else).
__device__ __forceinline__ void report_mismatch(int* __restrict__ fault, int which, int expected, int found)
{
    __hip_atomic_store(fault + 1, which, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(fault + 2, expected, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(fault + 3, found, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(fault, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// kWide: the table is addressed with 64-bit global loads instead of 32-bit offsets into a buffer resource (tables of
// 4 GB and more, wide rows of 2^24 vertices and more); the lanes a buffer load would have sent out of range load row 0
// instead and their values are replaced by zeros when they are added.
template <int MODE, int TS, int U, bool kWide>
__global__ __launch_bounds__(kStreamBlock) void aggregate_stream_kernel(
    float* __restrict__ out, float* __restrict__ partial, const float* __restrict__ table,
    const int* __restrict__ scol, const int* __restrict__ erow, const int* __restrict__ cev,
    const int* __restrict__ wtail, const float* __restrict__ scale, const StreamHeader* __restrict__ header,
    int* __restrict__ fault, int generation, int num_wave_chunks, int num_events,
    int num_nodes, int num_partials, int chunks, unsigned ld_bytes, int width_out, int ld_out, unsigned table_bytes,
    unsigned pad_row)
{
    constexpr int TPW = kWave / TS;
    constexpr int kParts = 8 / U;                  // batches per step
    constexpr int kCevPerTeam = TS / 4;            // cev counts chunks of 32 slots; a team owns 8 * TS slots
    // per wave: where the sum of every piece that ends in its slots goes.  x, y: address of the target row's first
    // float (0: nowhere), z: the factor (the row's scale; 1 for a partial sum), w: floats the target row takes
    // (a partial sum is one table row wide) | bit 16 for a partial sum
    __shared__ u32x4 ev_list[kStreamWaves][kStreamEvents + 1];

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int team = lane / TS;
    const int tl = lane % TS;
    const int w = blockIdx.x * kStreamWaves + wave;
    if (w >= num_wave_chunks) return;                       // wave-uniform; the LDS rows are wave-private
    // the counts the host remembers must be those of the plan in memory (they are unless the plan's bytes were
    // replaced behind the library's back): a mismatch ends the kernel instead of indexing with the wrong sizes,
    // and leaves a mark that eppgcn_aggregation_status reports (the output of this call is not written)
    if (header_mismatch(header, generation, num_events, num_partials)) {
        if (w == 0 && lane == 0) report_mismatch(fault, 1, generation, header->generation);
        return;
    }
    u32x4* my_list = ev_list[wave];
    constexpr unsigned kPartialTarget = 0x10000u;
    const unsigned ld_floats = ld_bytes / 4u;
    auto target_of = [&](int r) {
        unsigned long long a;
        unsigned factor, floats;
        if (r < 0) {                                    // never out of range with a well-formed stream
            const unsigned at = static_cast<unsigned>(r) & 0x7fffffffu;
            a = at < static_cast<unsigned>(num_partials)
                    ? reinterpret_cast<unsigned long long>(partial) + static_cast<unsigned long long>(at) * ld_bytes : 0ull;
            factor = __float_as_uint(1.f);
            floats = ld_floats | kPartialTarget;
        } else {
            a = r < num_nodes ? reinterpret_cast<unsigned long long>(out) + static_cast<unsigned long long>(r) * ld_out * 4ull : 0ull;
            factor = __float_as_uint(scale[min(r, num_nodes - 1)]);
            floats = static_cast<unsigned>(width_out);
        }
        return u32x4{static_cast<unsigned>(a), static_cast<unsigned>(a >> 32), factor, floats};
    };

    // the wave's 512 slot ids, 8 per lane (streamed once: non-temporal)
    const u32x4* idp = reinterpret_cast<const u32x4*>(scol + static_cast<size_t>(w) * kStreamWave) + lane * 2;
    const u32x4 id_lo = __builtin_nontemporal_load(idp);
    const u32x4 id_hi = __builtin_nontemporal_load(idp + 1);
    const unsigned ids[8] = {id_lo.x, id_lo.y, id_lo.z, id_lo.w, id_hi.x, id_hi.y, id_hi.z, id_hi.w};
    const int c0 = w * (kStreamWave / 32);
    const int ce_team = cev[c0 + team * kCevPerTeam];
    const int ce_first = cev[c0];
    const int ce_last = cev[c0 + kStreamWave / 32];
    const int tail_at = wtail[w];

    const __amdgpu_buffer_rsrc_t rows = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(table), 0,
                                                                          static_cast<int>(table_bytes), 0x00020000);
    const unsigned lane_off = tl < chunks ? static_cast<unsigned>(tl) * 16u : kNoRowOffset;
    const unsigned row_step = static_cast<unsigned>(__builtin_ctz(ld_bytes));       // wave-uniform

    // batch (s, part): the ids come from lane s of the team, registers part * U ...
    auto issue = [&](StreamBatch<U>& b, int s, auto part) {
        constexpr int kPart = decltype(part)::value;
        const int src = team * TS + s;
#pragma unroll
        for (int u = 0; u < U; ++u) b.c[u] = static_cast<unsigned>(__shfl(static_cast<int>(ids[kPart * U + u]), src, kWave));
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const unsigned id = swizzled_row(b.c[u] & 0x7fffffffu);      // the table's row order (common.hpp)
            // rows of a narrow team are a power of two bytes apart (row_step = log2): a shift serves any row count
            // of a table below 4 GB; wider rows use the 24-bit multiply (the host checks the row count)
            if constexpr (kWide) {
                const bool ok = lane_off != kNoRowOffset && id < pad_row;
                const unsigned long long off = static_cast<unsigned long long>(id) * ld_bytes + lane_off;
                b.v[u] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(table) + (ok ? off : 0ull));
            } else {
                unsigned row_off;
                if constexpr (TS <= kStreamShiftTeams) row_off = id << row_step;
                else row_off = __umul24(id, ld_bytes);
                const unsigned off = lane_off == kNoRowOffset ? kNoRowOffset : row_off + lane_off;
                b.v[u] = __builtin_amdgcn_raw_buffer_load_b128(rows, off, 0, 0);
            }
        }
    };
    using P0 = std::integral_constant<int, 0>;
    using P1 = std::integral_constant<int, kParts - 1>;

    StreamBatch<U> ba, bb;
    issue(ba, 0, P0{});            // the first gathers are under way while the piece list is staged

    // pieces that end in the wave's slots: [ev0, ev1)
    const int ev0 = ce_first & 0x7fffffff;
    const int ev1 = ce_last & 0x7fffffff;
    {
        const int staged = min(min(ev1, num_events) - ev0, kStreamEvents);
        for (int j = lane; j < staged; j += kWave) my_list[j] = target_of(erow[ev0 + j]);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }

    // a complete piece goes to its row, scaled; anything else, unscaled (factor 1), to its place among the partial
    // sums, where the whole pitch is written (lanes past the row's vectors hold zeros): a partial sum then fills its
    // 64- or 128-byte line and goes to memory without a read-modify-write
    auto flush = [&](const float (&a)[4], const u32x4& e) {
        const unsigned long long addr = static_cast<unsigned long long>(e.x) | (static_cast<unsigned long long>(e.y) << 32);
        if (addr == 0ull) return;
        float* dst = reinterpret_cast<float*>(addr) + tl * 4;
        const float f = __uint_as_float(e.z);
        const float v[4] = {a[0] * f, a[1] * f, a[2] * f, a[3] * f};
        if constexpr (MODE == kStoreExact) {
            store_row_floats<kStoreExact>(dst, v, 4);
        } else {
            const int n = static_cast<int>(e.w & 0xffffu) - tl * 4;
            if (e.w & kPartialTarget) store_row_floats<kStoreVec4>(dst, v, n);
            else store_row_floats<MODE>(dst, v, n);
        }
    };

    int ev = min(max((ce_team & 0x7fffffff) - ev0, 0), kStreamEvents);   // the team's next piece end in the staged list
    bool head_pending = ce_team < 0;             // the first piece end of the team closes a piece from an earlier team
    bool had_event = false;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    float head[4] = {0.f, 0.f, 0.f, 0.f};
    u32x4 head_to = {0u, 0u, 0u, 0u};
    u32x4 next_to = my_list[ev];

    auto consume = [&](const StreamBatch<U>& b) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            u32x4 v = b.v[u];
            if constexpr (kWide) {          // what a buffer load would have returned as zeros
                const bool ok = lane_off != kNoRowOffset && swizzled_row(b.c[u] & 0x7fffffffu) < pad_row;
                if (!ok) v = u32x4{0u, 0u, 0u, 0u};
            }
            acc[0] += __uint_as_float(v.x);
            acc[1] += __uint_as_float(v.y);
            acc[2] += __uint_as_float(v.z);
            acc[3] += __uint_as_float(v.w);
            if (static_cast<int>(b.c[u]) < 0) {            // the slot ends a piece
                if (head_pending) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) head[j] = acc[j];
                    head_to = next_to;
                    head_pending = false;
                } else {
                    flush(acc, next_to);
                }
                had_event = true;
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[j] = 0.f;
                ev = min(ev + 1, kStreamEvents);
                next_to = my_list[ev];
            }
        }
    };

    // two batches in flight; the loop bodies issue unconditionally so that the waits can count on the younger batch
    if constexpr (kParts == 2) {
        for (int s = 0; s + 1 < TS; ++s) {
            issue(bb, s, P1{});
            consume(ba);
            issue(ba, s + 1, P0{});
            consume(bb);
        }
        issue(bb, TS - 1, P1{});
        consume(ba);
        consume(bb);
    } else {
        for (int s = 0; s + 2 < TS; s += 2) {
            issue(bb, s + 1, P0{});
            consume(ba);
            issue(ba, s + 2, P0{});
            consume(bb);
        }
        issue(bb, TS - 1, P0{});
        consume(ba);
        consume(bb);
    }

    // ---- combine across the teams of the wave.  Inclusive segmented scan of the tails: a team in which a piece
    // ended starts a new segment (what came before it does not pass through it).
    float run[4] = {acc[0], acc[1], acc[2], acc[3]};
    bool stop = had_event;
    if constexpr (TPW > 1) {
#pragma unroll
        for (int d = 1; d < TPW; d <<= 1) {
            const bool take = team >= d && !stop;
            const int other_stop = __shfl_up(static_cast<int>(stop), d * TS, kWave);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float o = __shfl_up(run[j], d * TS, kWave);
                if (take) run[j] += o;
            }
            if (team >= d) stop = stop || other_stop != 0;
        }
    }
    // what flows into a team is the scan value of the team before it
    float carry[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float o = TPW > 1 ? __shfl_up(run[j], TS, kWave) : 0.f;
        carry[j] = team > 0 ? o : 0.f;
    }
    if (ce_team < 0 && had_event) {
#pragma unroll
        for (int j = 0; j < 4; ++j) head[j] += carry[j];
        flush(head, head_to);
    }
    // the wave's last tail belongs to a piece that ends in a later wave: one more partial sum
    if (team == TPW - 1 && tail_at >= 0) flush(run, target_of(tail_at | static_cast<int>(kStreamFlag)));
}

// Rows with partial sums: out[frow[i], :] = s[frow[i]] * (sum of the partial rows fptr[i] .. fptr[i+1]), summed in
// a fixed order, so the result does not depend on the order in which the waves of the stream kernel ran.  A wave
// takes 64 / TS rows.  Short lists: a team of TS lanes per row walks its list.  Rows with more than kFixTeamMax
// partial sums (hub rows cut into column blocks and waves) are then taken one at a time by the whole wave: team t
// adds the partial sums t, t + TPW, ..., and the teams are summed with cross-lane operations.
constexpr int kFixTeamMax = 32;
template <int MODE, int TS>
__global__ __launch_bounds__(256) void stream_fixup_kernel(float* __restrict__ out, const float* __restrict__ partial,
                                                           const int* __restrict__ frow, const int* __restrict__ fptr,
                                                           const float* __restrict__ scale, const StreamHeader* header,
                                                           int* __restrict__ fault, int generation,
                                                           int num_partials, int chunks, unsigned ld_bytes,
                                                           int width_out, int ld_out)
{
    constexpr int TPW = kWave / TS;
    if (header_mismatch(header, generation, -1, num_partials)) {              // same rule as the stream kernel
        if (blockIdx.x == 0 && threadIdx.x == 0) report_mismatch(fault, 2, generation, header->generation);
        return;
    }
    const int num_fix = header->num_fix;
    const int lane = threadIdx.x & (kWave - 1);
    const int team = lane / TS;
    const int tl = lane % TS;
    const long long wave0 = static_cast<long long>(blockIdx.x) * (256 / kWave) + threadIdx.x / kWave;
    const long long waves = static_cast<long long>(gridDim.x) * (256 / kWave);
    const char* base = reinterpret_cast<const char*>(partial) + tl * 16;
    // sixteen row loads in flight (most rows have fewer partial sums: one round trip), none of them behind a
    // branch of its own (an index past the end is replaced by a valid one and its row by zeros).  Plain loads: the
    // replaced indices re-read one row and the two halves of a 128-byte line are read by different instructions, both
    // of which the caches serve (non-temporal loads here cost 20 us per launch at R-MAT 22)
    constexpr int kFixLoads = 16;
    auto add_range = [&](float (&acc)[4], int beg, int end, int step) {
        if (tl >= chunks) return;
        for (int k = beg; k < end; k += kFixLoads * step) {
            f32x4 v[kFixLoads];
#pragma unroll
            for (int u = 0; u < kFixLoads; ++u) {
                const bool ok = k + u * step < end;
                v[u] = *reinterpret_cast<const f32x4*>(base + static_cast<size_t>(ok ? k + u * step : k) * ld_bytes);
                if (!ok) v[u] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int u = 0; u < kFixLoads; ++u) { acc[0] += v[u].x; acc[1] += v[u].y; acc[2] += v[u].z; acc[3] += v[u].w; }
        }
    };
    auto write_row = [&](const float (&acc)[4], int r, float s) {
        const float v[4] = {acc[0] * s, acc[1] * s, acc[2] * s, acc[3] * s};
        store_row_floats<MODE>(out + static_cast<size_t>(r) * ld_out + tl * 4, v, width_out - tl * 4);
    };
    for (long long wv = wave0; wv * TPW < num_fix; wv += waves) {
        const long long i = wv * TPW + team;
        const bool have = i < num_fix;
        const int r = have ? frow[i] : 0;
        const int beg = have ? fptr[i] : 0, end = have ? fptr[i + 1] : 0;
        // short lists: every team its own row; then the long ones, one at a time, by the whole wave
        const bool is_long = end - beg > kFixTeamMax;
        const float s_row = have ? scale[r] : 0.f;      // under way while the partial sums are read
        if (!is_long) {
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
            add_range(acc, beg, end, 1);
            if (have) write_row(acc, r, s_row);
        }
        uint64_t longs = __ballot(is_long && tl == 0);
        while (longs) {                                 // wave-uniform
            const int lead = __builtin_ctzll(longs);
            longs &= longs - 1;
            const int rb = __shfl(beg, lead, kWave), re = __shfl(end, lead, kWave), rr = __shfl(r, lead, kWave);
            const float rs = __shfl(s_row, lead, kWave);
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
            add_range(acc, rb + team, re, TPW);
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] = cross_team_sum<TS>(acc[j]);
            if (team == 0) write_row(acc, rr, rs);
        }
    }
}

// ---------------------------------------------------------------- the mark of a header mismatch
static __device__ __align__(16) int plan_fault_words[kPlanFaultWords];
}  // namespace eppgcn

#include <atomic>
#include <map>
#include <mutex>

namespace eppgcn {
static std::mutex g_fault_mutex;
static std::map<int, int*> g_fault_address;     // per device: each GPU holds its own copy of the words

int plan_fault_address(int** words)
{
    int device = 0;
    EPPGCN_HIP(hipGetDevice(&device));
    std::lock_guard<std::mutex> lock(g_fault_mutex);
    auto it = g_fault_address.find(device);
    if (it == g_fault_address.end()) {
        void* p = nullptr;
        EPPGCN_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(plan_fault_words)));
        it = g_fault_address.emplace(device, static_cast<int*>(p)).first;
    }
    *words = it->second;
    return kOk;
}

// process-wide knobs (tuning header): atomics, so that a setter racing with a call is at least not a data race
static std::atomic<int> g_stream_mode{1};
static std::atomic<bool> g_force_wide_stream{false};     // tests: the 64-bit addressing variant at any size
void set_stream_mode(int on) { g_stream_mode.store(on ? 1 : 0); g_force_wide_stream.store(on == 2); }

// Team size for rows of `chunks` 16-byte vectors, 0 when the stream kernel does not cover the shape.
static int stream_team(int chunks)
{
    int ts = 4;
    while (ts < 64 && ts < chunks) ts <<= 1;
    return chunks <= 64 ? ts : 0;
}

// Does the shape need 64-bit addressing?  32-bit byte offsets cover tables below 4 GB; teams of up to kStreamShiftTeams
// lanes turn a row into a byte offset with a shift (rows a power of two bytes apart: the workspace's pitch for such
// widths), wider teams multiply 24-bit operands.
static bool stream_needs_wide(int num_nodes, int dim, int ld_in)
{
    const unsigned long long bytes = static_cast<unsigned long long>(swizzle_padded_rows(num_nodes)) * ld_in * 4ull;
    if (bytes + 16 >= (1ull << 32)) return true;
    if (stream_team((dim + 3) / 4) <= kStreamShiftTeams) return (ld_in & (ld_in - 1)) != 0;
    return !(swizzle_padded_rows(num_nodes) < (1 << 24) && ld_in * 4 < (1 << 24));
}

// Can a launch over a pre-scaled table with rows of ld_in floats run through the stream kernel?
bool stream_covers(int num_nodes, int dim, int ld_in, const float* table)
{
    if (!g_stream_mode.load() || force_wide_index()) return false;
    if (ld_in % 4 != 0 || reinterpret_cast<uintptr_t>(table) % 16 != 0) return false;
    if (stream_team((dim + 3) / 4) == 0 || (dim + 3) / 4 * 4 > ld_in) return false;
    return swizzle_padded_rows(num_nodes) < (1ll << 31);
}

// Stream kernel + fix-up kernel over a pre-scaled table in swizzled row order (stream_covers() holds).  `partial` holds
// info.header.num_partials rows of ld_in floats.  Rows without slots are not written (the caller clears them).
int launch_aggregate_stream(float* out, float* partial, const float* table, const int* scol, const StreamView& sv,
                            const StreamInfo& info, const float* scale, int num_nodes, int dim, int ld_in,
                            hipStream_t stream)
{
    const int chunks = (dim + 3) / 4;
    const int ts = stream_team(chunks);
    const long long padded = stream_padded_slots(info.num_slots);
    const bool wide = stream_needs_wide(num_nodes, dim, ld_in) || g_force_wide_stream.load();
    const unsigned long long bytes = wide ? 0ull : static_cast<unsigned long long>(swizzle_padded_rows(num_nodes)) * ld_in * 4ull;
    const unsigned pad_row = static_cast<unsigned>(swizzle_padded_rows(num_nodes));
    const int num_wave_chunks = static_cast<int>(padded / kStreamWave);
    if (num_wave_chunks == 0) return kOk;
    const dim3 grid((num_wave_chunks + kStreamWaves - 1) / kStreamWaves), block(kStreamBlock);
    const uintptr_t a = reinterpret_cast<uintptr_t>(out);
    const int mode = (dim % 4 == 0 && a % 16 == 0) ? ((dim == ts * 4 && ld_in == ts * 4) ? kStoreExact : kStoreVec4) : kStorePlain;
    const int num_fix = info.header.num_fix;
    long long fix_blocks = (static_cast<long long>(num_fix) * ts + 255) / 256;
    if (fix_blocks > 256 * 64) fix_blocks = 256 * 64;
    const dim3 fgrid(static_cast<unsigned>(fix_blocks < 1 ? 1 : fix_blocks));
    int* fault = nullptr;
    if (int rc = plan_fault_address(&fault)) return rc;
#define EPPGCN_STREAM_KERNEL(MODE_, TS_, WIDE_)                                                                        \
    hipLaunchKernelGGL((aggregate_stream_kernel<MODE_, TS_, 8, WIDE_>), grid, block, 0, stream, out, partial, table,   \
                       scol, sv.erow, sv.cev, sv.wtail, scale, sv.header, fault, info.header.generation,              \
                       num_wave_chunks, info.header.num_events,                                                       \
                       num_nodes, info.header.num_partials, chunks, static_cast<unsigned>(ld_in) * 4u, dim, dim,      \
                       static_cast<unsigned>(bytes), pad_row)
#define EPPGCN_STREAM(MODE_, TS_)                                                                                      \
    do {                                                                                                              \
        if (wide) EPPGCN_STREAM_KERNEL(MODE_, TS_, true);                                                              \
        else EPPGCN_STREAM_KERNEL(MODE_, TS_, false);                                                                  \
        if (num_fix > 0)                                                                                              \
            hipLaunchKernelGGL((stream_fixup_kernel<MODE_, TS_>), fgrid, dim3(256), 0, stream, out, partial, sv.frow,  \
                               sv.fptr, scale, sv.header, fault, info.header.generation,                              \
                               info.header.num_partials, chunks,                                                      \
                               static_cast<unsigned>(ld_in) * 4u, dim, dim);                                          \
    } while (0)
#define EPPGCN_STREAM_TS(MODE_)                                                                                        \
    do {                                                                                                              \
        switch (ts) {                                                                                                 \
            case 4: EPPGCN_STREAM(MODE_, 4); break;                                                                    \
            case 8: EPPGCN_STREAM(MODE_, 8); break;                                                                    \
            case 16: EPPGCN_STREAM(MODE_, 16); break;                                                                  \
            case 32: EPPGCN_STREAM(MODE_, 32); break;                                                                  \
            default: EPPGCN_STREAM(MODE_, 64); break;                                                                  \
        }                                                                                                             \
    } while (0)
    if (mode == kStoreExact) EPPGCN_STREAM_TS(kStoreExact);
    else if (mode == kStoreVec4) EPPGCN_STREAM_TS(kStoreVec4);
    else EPPGCN_STREAM_TS(kStorePlain);
#undef EPPGCN_STREAM_TS
#undef EPPGCN_STREAM
#undef EPPGCN_STREAM_KERNEL
    EPPGCN_HIP(hipGetLastError());
    return kOk;
}

}  // namespace eppgcn
