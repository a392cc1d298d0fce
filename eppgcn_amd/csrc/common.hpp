// Shared device helpers for the gfx950 (CDNA4, wave64) kernels of the GCN
// aggregation path: cross-lane primitives, the decoupled look-back tile
// protocol, and host-side error plumbing.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>

namespace eppgcn {

constexpr int kWave = 64;

// ---------------------------------------------------------------- host errors
// Every C entry point returns 0 on success or a negative code and leaves a
// message readable through eppgcn_last_error().
enum : int {
    kOk = 0,
    kErrInvalidArgument = -1,
    kErrHip = -2,
    kErrScanStalled = -3,   // a look-back wait exceeded its spin limit
    kErrCapacity = -4,      // an output buffer was too small for the result
    kErrPlanMismatch = -5,  // the memory at a plan's address does not hold the plan the library knows there
};

void set_error(const std::string& msg);
int hip_fail(hipError_t e, const char* what);

#define EPPGCN_HIP(expr)                                        \
    do {                                                        \
        hipError_t _e = (expr);                                 \
        if (_e != hipSuccess) return ::eppgcn::hip_fail(_e, #expr); \
    } while (0)

#define EPPGCN_REQUIRE(cond, msg)                               \
    do {                                                        \
        if (!(cond)) {                                          \
            ::eppgcn::set_error(std::string(__func__) + ": " + (msg)); \
            return ::eppgcn::kErrInvalidArgument;               \
        }                                                       \
    } while (0)

// Zeroes `words` 32-bit words at p (4-byte aligned) with a fill kernel.  Used instead of
// hipMemsetAsync everywhere so that every call of the library can be captured into a HIP graph
// (memset nodes are the one node kind callers are told to avoid on this platform).
int launch_zero_words(void* p, size_t words, hipStream_t stream);
// The streaming helper kernels index with 32 bits when the element count allows; true forces their
// 64-bit instantiations at any size (so that tests reach them without 16 GB matrices).
bool force_wide_index();
void set_force_wide_index(bool on);
// Zeroes the rows of out[num_rows, dim] whose bit in `skip` is clear (rows with a set bit are left as they are).
int launch_zero_rows_unless(float* out, const uint32_t* skip, long long num_rows, int dim, hipStream_t stream);

// ---------------------------------------------------------------- execution plan layout
// One caller-owned buffer: ptr[P+1] | row[P] | flags[P] | single[ceil(N/32)] | col[S_pad] | stream form, each
// part 256-byte aligned (contents described in schedule.hip).  Offsets depend on the group count, the
// slot count and the vertex count alone.
struct PlanView {
    int* ptr;
    int* row;
    uint8_t* flags;
    uint32_t* single;   // bit r: row r consists of exactly one non-empty group (it is written by one plain store)
    int* col;           // column ids in processing order; bit 31 marks the last slot of a piece (see below)
};

// Stream form of a plan (read by stream.hip, built by schedule.hip).  A "piece" is a maximal stretch of
// plan entries that continue one another, i.e. consecutive slots of one row.
constexpr int kStreamWave = 512;     // slots a wave of the stream kernel takes
constexpr int kStreamChunk = 32;     // piece ends are counted per chunk of this many slots
constexpr unsigned kStreamFlag = 0x80000000u;
constexpr int kStreamIdMask = 0x7fffffff;
constexpr int kPlanMagic = 0x45505047;   // "EPPG"
struct StreamHeader {
    int valid;          // 1: the stream arrays describe the plan (0: groups were empty or a scan stalled)
    int num_events;     // pieces
    int num_partials;   // partial sums the stream kernel leaves for the fix-up kernel
    int num_fix;        // rows the fix-up kernel writes
    int empty_rows;     // rows without any slot (the output clear zeroes them)
    int error;          // a look-back scan of the build stalled
    int empty_groups;   // != 0: the plan holds empty groups (no stream form)
    int magic;          // kPlanMagic: the build got as far as writing the header
    int generation;     // number of the build in this process (> 0); the host remembers it with the counts
    int num_parts;      // the sizes the plan was built with (its layout depends on them)
    int num_nodes;
    int num_slots;
    int pad[4];
};
static_assert(sizeof(StreamHeader) == 64, "header layout");
struct StreamView {
    StreamHeader* header;
    int* erow;          // [P]  per piece: its row, or kStreamFlag | index of its partial sum
    int* cev;           // [S_pad / 32 + 1]  pieces that end before slot 32 c; bit 31: slot 32 c continues a piece
    int* wtail;         // [S_pad / 512]  index of the partial sum of what wave w holds at its end, or -1
    uint32_t* touched;  // [ceil(N/32)]  bit r: row r has at least one slot
    int* frow;          // [N]  rows with partial sums ...
    int* fptr;          // [N+1] ... and where their partial sums start
};
inline size_t plan_align(size_t x) { return (x + 255) / 256 * 256; }
inline size_t plan_single_words(long long num_nodes)
{
    return (static_cast<size_t>(num_nodes > 0 ? num_nodes : 0) + 31) / 32;
}
inline long long stream_padded_slots(long long num_slots)
{
    const long long s = num_slots > 0 ? num_slots : 0;
    return (s + kStreamWave - 1) / kStreamWave * kStreamWave;
}
inline size_t plan_groups_bytes(long long num_parts, long long num_slots, long long num_nodes)
{
    const size_t p = static_cast<size_t>(num_parts > 0 ? num_parts : 0);
    const size_t s = static_cast<size_t>(stream_padded_slots(num_slots));
    return plan_align(4 * (p + 1)) + plan_align(4 * p) + plan_align(p) + plan_align(4 * plan_single_words(num_nodes)) +
           plan_align(4 * s);
}
inline size_t plan_bytes(long long num_parts, long long num_slots, long long num_nodes)
{
    const size_t p = static_cast<size_t>(num_parts > 0 ? num_parts : 0);
    const size_t s = static_cast<size_t>(stream_padded_slots(num_slots));
    const size_t n = static_cast<size_t>(num_nodes > 0 ? num_nodes : 0);
    return plan_groups_bytes(num_parts, num_slots, num_nodes) + plan_align(sizeof(StreamHeader)) + plan_align(4 * p) +
           plan_align(4 * (s / kStreamChunk + 1)) + plan_align(4 * (s / kStreamWave)) +
           plan_align(4 * plan_single_words(num_nodes)) + plan_align(4 * n) + plan_align(4 * (n + 1));
}
inline PlanView plan_view(void* plan, long long num_parts, long long num_nodes)
{
    const size_t p = static_cast<size_t>(num_parts);
    char* b = static_cast<char*>(plan);
    PlanView v;
    v.ptr = reinterpret_cast<int*>(b);
    b += plan_align(4 * (p + 1));
    v.row = reinterpret_cast<int*>(b);
    b += plan_align(4 * p);
    v.flags = reinterpret_cast<uint8_t*>(b);
    b += plan_align(p);
    v.single = reinterpret_cast<uint32_t*>(b);
    b += plan_align(4 * plan_single_words(num_nodes));
    v.col = reinterpret_cast<int*>(b);
    return v;
}
inline StreamView stream_view(void* plan, long long num_parts, long long num_slots, long long num_nodes)
{
    const size_t p = static_cast<size_t>(num_parts > 0 ? num_parts : 0);
    const size_t s = static_cast<size_t>(stream_padded_slots(num_slots));
    const size_t n = static_cast<size_t>(num_nodes > 0 ? num_nodes : 0);
    char* b = static_cast<char*>(plan) + plan_groups_bytes(num_parts, num_slots, num_nodes);
    StreamView v;
    v.header = reinterpret_cast<StreamHeader*>(b);
    b += plan_align(sizeof(StreamHeader));
    v.erow = reinterpret_cast<int*>(b);
    b += plan_align(4 * p);
    v.cev = reinterpret_cast<int*>(b);
    b += plan_align(4 * (s / kStreamChunk + 1));
    v.wtail = reinterpret_cast<int*>(b);
    b += plan_align(4 * (s / kStreamWave));
    v.touched = reinterpret_cast<uint32_t*>(b);
    b += plan_align(4 * plan_single_words(num_nodes));
    v.frow = reinterpret_cast<int*>(b);
    b += plan_align(4 * n);
    v.fptr = reinterpret_cast<int*>(b);
    return v;
}
// Row order of a separate pre-scaled feature table.  Vertex ids of graphs with a recursive (Kronecker / R-MAT)
// structure are biased towards few set bits, so the hot rows of a table laid out by id share their low address
// bits and their gathers pile up on a few memory channels (measured at R-MAT scale 22: 8 % of the kernel time).
// Row r therefore lives at index r ^ ((r >> 5) & 4095): a permutation inside every aligned block of 4096 rows,
// which keeps a column block of the plan one contiguous range of the table.
constexpr unsigned kRowSwizzleShift = 5;
constexpr unsigned kRowSwizzleMask = 4095;
__host__ __device__ inline unsigned swizzled_row(unsigned r, unsigned mask = kRowSwizzleMask)
{
    return r ^ ((r >> kRowSwizzleShift) & mask);
}
// rows a swizzled table of num_nodes vertices spans (whole blocks)
__host__ __device__ inline long long swizzle_padded_rows(long long num_nodes)
{
    const long long n = num_nodes > 0 ? num_nodes : 0;
    return (n + kRowSwizzleMask) / (kRowSwizzleMask + 1) * (kRowSwizzleMask + 1);
}

// What the host knows about a plan's stream form once eppgcn_plan_status has read its header.
struct StreamInfo {
    long long num_parts, num_slots, num_nodes;
    StreamHeader header;
};
// nullptr when the plan at this address has no (known) stream form
const StreamInfo* find_stream_info(const void* plan, StreamInfo* copy);
void forget_stream_info(const void* plan);
void remember_stream_info(const void* plan, const StreamInfo& info);
// Device words (one set per GPU, inside the library) in which the stream and fix-up kernels leave a mark when
// the plan header in memory is not the one the host remembers for that address: [0] != 0 says so, [1] which kernel
// saw it (1 stream, 2 fix-up), [2] / [3] the build number the host expected / the one found.  The address on the
// current device; looked up once per device (eppgcn_plan_status does it, so never under a graph capture).
constexpr int kPlanFaultWords = 4;
int plan_fault_address(int** words);

// ---------------------------------------------------------------- kernel timers
// Optional event timing of the kernels of one call (off by default: calls stay
// asynchronous).  When enabled the destructor synchronises on the stop event and
// adds the elapsed milliseconds to the sinks.
bool timing_enabled();
// Accumulators (ms) of the passes an aggregation call runs before its kernel: 0 = output clear,
// 1 = pre-scaling of the input into the feature workspace.
double* phase_sink(int which);
struct KernelTimer {
    hipStream_t stream;
    double* sink;
    double* sink2;
    hipEvent_t start = nullptr, stop = nullptr;
    KernelTimer(hipStream_t s, double* a, double* b = nullptr) : stream(s), sink(a), sink2(b)
    {
        if (!a || !timing_enabled()) return;
        if (hipEventCreate(&start) != hipSuccess) { start = nullptr; return; }
        if (hipEventCreate(&stop) != hipSuccess) { (void)hipEventDestroy(start); start = nullptr; return; }
        (void)hipEventRecord(start, stream);
    }
    ~KernelTimer()
    {
        if (!start) return;
        float ms = 0.f;
        if (hipEventRecord(stop, stream) == hipSuccess && hipEventSynchronize(stop) == hipSuccess &&
            hipEventElapsedTime(&ms, start, stop) == hipSuccess) {
            *sink += ms;
            if (sink2) *sink2 += ms;
        }
        (void)hipEventDestroy(start);
        (void)hipEventDestroy(stop);
    }
    KernelTimer(const KernelTimer&) = delete;
    KernelTimer& operator=(const KernelTimer&) = delete;
};

// ---------------------------------------------------------------- lane helpers
__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

// Number of set ballot bits strictly below this lane (rank of the lane among the
// lanes whose predicate held).
__device__ __forceinline__ int ballot_rank(uint64_t ballot)
{
    return __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(ballot >> 32),
                                     __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(ballot), 0u));
}

// A wave looks at 64 consecutive rows (lane l at row base + l, `wanted` says whether the row needs
// work) and leaves the wanted rows, in order, in its own 64-entry LDS list; returns how many.  The
// barriers order the LDS traffic of the wave's lanes (the list is private to the wave).
__device__ __forceinline__ int compact_wanted_rows(int* __restrict__ list, unsigned row, bool wanted)
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");     // earlier reads of the list are done
    __builtin_amdgcn_wave_barrier();
    const uint64_t m = __ballot(wanted);
    if (wanted) list[ballot_rank(m)] = static_cast<int>(row);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    return __popcll(m);
}

// DPP controls (GFX9 encoding): row_ror:n rotates within a row of 16 lanes.
constexpr int kDppRowRor4 = 0x124;
constexpr int kDppRowRor8 = 0x128;
constexpr int kDppQuadXor1 = 0xB1;   // quad_perm [1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;   // quad_perm [2,3,0,1]

template <int kCtrl>
__device__ __forceinline__ float dpp_f32(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), kCtrl, 0xF, 0xF, false));
}

// value of lane (l ^ 16) inside each half of 32 lanes: ds_swizzle bit-mask mode,
// and_mask = 0x1F, or_mask = 0, xor_mask = 0x10.
__device__ __forceinline__ float swizzle_xor16(float v)
{
    return __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), 0x401F));
}

// Sum of v over the lanes that hold the same position inside their team, for
// teams of kTeam consecutive lanes: afterwards every lane holds the total of the
// 64/kTeam lanes congruent to it modulo kTeam.  Offsets below 16 stay inside a
// DPP row (rotations), 16 uses ds_swizzle, 32 a bpermute: no LDS memory and no
// global atomics are involved.
template <int kTeam>
__device__ __forceinline__ float cross_team_sum(float v)
{
    if constexpr (kTeam <= 1) v += dpp_f32<kDppQuadXor1>(v);
    if constexpr (kTeam <= 2) v += dpp_f32<kDppQuadXor2>(v);
    if constexpr (kTeam <= 4) v += dpp_f32<kDppRowRor4>(v);
    if constexpr (kTeam <= 8) v += dpp_f32<kDppRowRor8>(v);
    if constexpr (kTeam <= 16) v += swizzle_xor16(v);
    if constexpr (kTeam <= 32) v += __shfl_xor(v, 32, kWave);
    return v;
}

__device__ __forceinline__ int wave_inclusive_scan(int v)
{
    const int lane = lane_id();
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        int t = __shfl_up(v, off, kWave);
        if (lane >= off) v += t;
    }
    return v;
}

__device__ __forceinline__ uint64_t wave_inclusive_scan_u64(uint64_t v)
{
    const int lane = lane_id();
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        uint64_t t = static_cast<uint64_t>(__shfl_up(static_cast<long long>(v), off, kWave));
        if (lane >= off) v += t;
    }
    return v;
}

__device__ __forceinline__ uint64_t wave_sum_u64(uint64_t v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1)
        v += static_cast<uint64_t>(__shfl_xor(static_cast<long long>(v), off, kWave));
    return v;
}

// ---------------------------------------------------------------- look-back tiles
// One 64-bit descriptor per tile: status in the two top bits, payload below.
// Status and payload travel in one relaxed agent-scope atomic, so a reader that
// sees the status also sees the payload.  Payloads are sums of non-negative
// fields that never carry into each other, so packed payloads add directly.
constexpr uint64_t kTileEmpty = 0;
constexpr uint64_t kTileAggregate = 1ull << 62;
constexpr uint64_t kTilePrefix = 2ull << 62;
constexpr uint64_t kTilePayloadMask = (1ull << 62) - 1;
constexpr unsigned kSpinLimit = 1u << 22;   // polls before a wait is declared stalled

struct ScanState {
    int counter;        // next tile id to hand out
    int error;          // set to 1 when a look-back wait hit its spin limit
    int counts[2];      // results the last tile publishes (meaning depends on the kernel)
    int overflow;       // set to 1 when an output would not fit its capacity
    int pad[3];
};
// Scan mode, a kernel argument of every scan kernel (it stays in scalar registers: the ScanState line is
// hammered by the tile-id atomics, so nothing else is read from it per tile): the low 31 bits are the
// number of polls before a wait is declared stalled (0 = kSpinLimit); the top bit is the test mode in
// which tile 0 never publishes, so that every look-back ends in a bounded stall.  The host value sits
// behind a test knob.
unsigned scan_mode();
void set_scan_test_mode(unsigned spin_limit, int mute_first_tile);
static_assert(sizeof(ScanState) == 32, "descriptor array starts 32 bytes into the workspace");

__device__ __forceinline__ void tile_store(uint64_t* desc, int tile, uint64_t v)
{
    __hip_atomic_store(desc + tile, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ uint64_t tile_load(uint64_t* desc, int tile)
{
    return __hip_atomic_load(desc + tile, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Block-wide dynamic tile id.  Ids are handed out in start order, so when tile t
// runs every tile below t is already running or finished: waiting on them cannot
// deadlock on hardware that keeps resident workgroups running.
__device__ __forceinline__ int acquire_tile(ScanState* st, int* s_tile)
{
    if (threadIdx.x == 0) *s_tile = atomicAdd(&st->counter, 1);
    __syncthreads();
    return *s_tile;
}

// Executed by one full wave.  Publishes this tile's aggregate, walks back over
// the predecessors 64 at a time until a tile with a known inclusive prefix is
// found, publishes this tile's inclusive prefix and returns its exclusive prefix
// to every lane.  Every wait is bounded: after the spin limit the error flag is
// raised and the walk continues with what it has, so the kernel always drains.
__device__ __forceinline__ uint64_t tile_lookback(uint64_t* desc, ScanState* st, int tile, uint64_t aggregate,
                                                  unsigned mode)
{
    const int lane = lane_id();
    if (tile == 0) {
        if (lane == 0 && (mode >> 31) == 0) tile_store(desc, 0, kTilePrefix | aggregate);
        return 0;
    }
    const unsigned spin_limit = (mode & 0x7fffffffu) ? (mode & 0x7fffffffu) : kSpinLimit;
    if (lane == 0) tile_store(desc, tile, kTileAggregate | aggregate);
    uint64_t exclusive = 0;
    int base = tile - 1;
    bool stalled = false;
    while (true) {
        const int t = base - lane;
        uint64_t d = kTilePrefix;               // tiles before the first count as "prefix 0"
        unsigned spins = 0;
        while (true) {
            if (t >= 0) d = tile_load(desc, t);
            const bool ready = (d >> 62) != 0;
            if (__all(ready)) break;
            if (++spins >= spin_limit) { stalled = true; break; }
            __builtin_amdgcn_s_sleep(1);
        }
        const uint64_t has_prefix = __ballot((d >> 62) == 2);
        const int first = has_prefix ? __builtin_ctzll(has_prefix) : kWave;
        exclusive += wave_sum_u64(lane <= first ? (d & kTilePayloadMask) : 0ull);
        if (first < kWave || stalled) break;
        base -= kWave;
    }
    if (lane == 0) {
        if (stalled) atomicExch(&st->error, 1);
        tile_store(desc, tile, kTilePrefix | ((exclusive + aggregate) & kTilePayloadMask));
    }
    return exclusive;
}

}  // namespace eppgcn
