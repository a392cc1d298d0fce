// Neighbour-group aggregation for gfx950 (wave64): forward SpMM, unpruned
// backward SpMM and the pruned backward that walks the compacted execution path.
//
// Replaces the reference's spmm_forward_cuda_kernel / spmm_backward_cuda_kernel
// (EPPGCN/GCNConv/EPPGCN_kernel.cu:204-295, :471-545) and ours_backward_cuda_kernel
// (:626-670).  Same contract, different machine mapping:
//
//   out[r, :] = sum over the slots e of every group of row r of
//               s[r] * s[col[e]] * in[col[e], :]
//
// Mapping.  A wave of 64 lanes is cut into teams of TS lanes; a team owns one
// neighbour group and its lanes stripe the feature row in contiguous vectors of
// VW floats (lane l of the team holds columns [l*VW, l*VW+VW), then +TS*VW ...),
// so one gather instruction fetches 64/TS whole neighbour rows with contiguous
// bytes per row.  The groups of a wave are consecutive, hence their CSR slots are
// one contiguous range: the wave first stages that range coalesced into LDS,
// which turns the per-neighbour dependent chain "id -> row" into batched phases
// with many requests in flight.  Partial sums live in registers.
//
// Neighbour scale.  Gathering s[col[e]] per edge costs one extra random memory
// request per edge (measured: a quarter of the kernel time at width 16).  With a
// workspace the features are scaled once per call (ws[c,:] = s[c]*in[c,:], one
// streaming pass) and the kernel gathers pre-scaled rows and multiplies by s[r]
// at the flush.  Without a workspace the kernel stages (id, scale) pairs and
// weights every row by fl32(s[r]*s[c]) as the reference does.  A pruned path that
// reads few rows (bitmap of the vertices in its edge list) scales only those.
//
// Output clear.  Rows summed with atomics, and rows without groups, must start
// at zero; a row that is one non-empty group is written whole by one store.  With
// a plan (which records those rows) only the former are cleared.
//
// Flush.  Groups of one row that sit in the same wave are first summed across
// teams in registers (DPP rotations / ds_swizzle when the whole wave is one row,
// a segmented shuffle reduction otherwise).  A row that lies entirely inside the
// wave is then written with plain stores; only rows spread over several waves
// use float atomics, once per wave instead of once per group.
// Precondition: the groups of one row are consecutive (build_part and the path
// splitter produce them that way).
#include <atomic>
#include <type_traits>

#include "common.hpp"

namespace eppgcn {

constexpr int kAggBlock = 256;
constexpr int kAggWaves = kAggBlock / kWave;
constexpr int kStageCap = 1024;  // slots of the staged window of a wave
// Staged slot s lives at LDS word s + s/32: teams read their groups at strides that are
// often a power of two (a backward group size of 32 puts all 16 teams of a wave on one bank);
// one pad word per 32 slots spreads such strides over the 32 banks.
constexpr int kStageWords = kStageCap + kStageCap / 32;
__device__ __forceinline__ int stage_index(int slot) { return slot + (slot >> 5); }

// ---------------------------------------------------------------- vectors
template <int VW> struct Vec;
template <> struct Vec<1> {
    float v[1];
    __device__ static Vec load(const float* p) { Vec r; r.v[0] = *p; return r; }
    __device__ void store(float* p) const { *p = v[0]; }
};
template <> struct Vec<2> {
    float v[2];
    __device__ static Vec load(const float* p)
    {
        float2 t = *reinterpret_cast<const float2*>(p);
        Vec r; r.v[0] = t.x; r.v[1] = t.y; return r;
    }
    // 8-byte pieces belong to rows that share their 64-byte sectors with their neighbours (width 22: 88-byte rows),
    // written by other teams at other times: plain stores, so that the cache puts the sectors together (rows of
    // 16-byte pieces below are whole sectors for the usual widths, written once: non-temporal)
    __device__ void store(float* p) const { *reinterpret_cast<float2*>(p) = make_float2(v[0], v[1]); }
};
template <> struct Vec<4> {
    float v[4];
    __device__ static Vec load(const float* p)
    {
        float4 t = *reinterpret_cast<const float4*>(p);
        Vec r; r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z; r.v[3] = t.w; return r;
    }
    __device__ void store(float* p) const
    {
        typedef float f4 __attribute__((ext_vector_type(4)));
        const f4 t = {v[0], v[1], v[2], v[3]};
        __builtin_nontemporal_store(t, reinterpret_cast<f4*>(p));
    }
};

// ---------------------------------------------------------------- group sources
// What the kernel asks about group p (p = position in processing order):
//   row_of       the row the group adds into
//   has_prev     the row has groups before this one that this position does not follow
//   has_next     ... after this one
//   joins_left   the group continues the group at position p-1 (same row, adjacent)
//   joins_right  the group at position p+1 continues this one
// For groups processed in their own order the two pairs coincide.

// Forward groups: (part_ptr, part2node) as build_part produces them.
struct ForwardGroups {
    const int* part_ptr;
    const int* part2node;
    __device__ int row_of(int p, int) const { return part2node[p]; }
    __device__ bool has_prev(int p, int row, int) const { return p > 0 && part2node[p - 1] == row; }
    __device__ bool has_next(int p, int row, int, int num_parts) const
    {
        return p + 1 < num_parts && part2node[p + 1] == row;
    }
    __device__ bool joins_left(int, bool prev) const { return prev; }
    __device__ bool joins_right(int, bool next) const { return next; }
};

// Backward groups over the compacted path: the row of a group is the id of its
// first kept edge (EPPGCN/GCNConv/EPPGCN_kernel.cu:642-646).
struct CompactedGroups {
    const int* part_ptr;
    const int* ids;
    __device__ int row_of(int, int gbeg) const { return ids[gbeg]; }
    __device__ bool has_prev(int, int row, int gbeg) const { return gbeg > 0 && ids[gbeg - 1] == row; }
    __device__ bool has_next(int p, int row, int gend, int num_parts) const
    {
        return p + 1 < num_parts && ids[gend] == row;
    }
    __device__ bool joins_left(int, bool prev) const { return prev; }
    __device__ bool joins_right(int, bool next) const { return next; }
};

// Groups of an execution plan: re-ordered copy with precomputed row and adjacency flags
// (bit0 has_prev, bit1 has_next, bit2 joins_left, bit3 joins_right; all in terms of the
// original group order, see schedule.hip).
struct PlanGroups {
    const int* part_ptr;
    const int* row;
    const uint8_t* flags;
    __device__ int row_of(int p, int) const { return row[p]; }
    __device__ bool has_prev(int p, int, int) const { return (flags[p] & 1) != 0; }
    __device__ bool has_next(int p, int, int, int) const { return (flags[p] & 2) != 0; }
    __device__ bool joins_left(int p, bool) const { return (flags[p] & 4) != 0; }
    __device__ bool joins_right(int p, bool) const { return (flags[p] & 8) != 0; }
};

// ---------------------------------------------------------------- pre-scaling pass
// dst[r, j] = scale[r] * src[r, j] for j < dim and 0 for dim <= j < ld_dst.  The destination
// row pitch ld_dst is a multiple of 4 floats, so every thread writes one aligned float4; rows
// padded to whole 32-byte sectors let the gather fetch fewer sectors per row and use 16-byte
// loads for widths such as 22 whose rows are only 8-byte aligned in the caller's layout.
//
// `rows` (optional): one bit per row; a row whose bit is clear is skipped (the caller knows that
// no group gathers it, e.g. the rows outside the kept path of a pruned backward), so the pass costs
// what the gathered rows cost.  Index: unsigned when the element count fits in 32 bits.
__device__ inline bool row_wanted(const uint32_t* __restrict__ rows, unsigned long long r)
{
    return rows == nullptr || ((rows[r >> 5] >> (r & 31)) & 1u) != 0;
}

template <class Index>
__global__ __launch_bounds__(256) void scale_rows_kernel(float* __restrict__ dst, const float* __restrict__ src,
                                                         const float* __restrict__ scale,
                                                         const uint32_t* __restrict__ rows, Index total_vecs,
                                                         Index vecs_per_row, Index dim, bool pairs, unsigned swz_mask)
{
    const Index stride = static_cast<Index>(gridDim.x) * blockDim.x;
    for (Index i = static_cast<Index>(blockIdx.x) * blockDim.x + threadIdx.x; i < total_vecs; i += stride) {
        const Index r = i / vecs_per_row;
        if (row_wanted(rows, r)) {
            const Index c0 = (i - r * vecs_per_row) * 4;
            // row r of the table lives at swizzled_row(r) (the mask is 0 for a table in vertex order)
            const size_t at = static_cast<size_t>(swizzled_row(static_cast<unsigned>(r), swz_mask)) * vecs_per_row * 4 + c0;
            const float s = scale[r];
            const float* row = src + static_cast<size_t>(r) * dim;
            float4 v;
            if (pairs) {                 // even width, 8-byte aligned source: a pair is all in or all out
                const float2 lo = c0 < dim ? *reinterpret_cast<const float2*>(row + c0) : make_float2(0.f, 0.f);
                const float2 hi = c0 + 2 < dim ? *reinterpret_cast<const float2*>(row + c0 + 2) : make_float2(0.f, 0.f);
                v = make_float4(s * lo.x, s * lo.y, s * hi.x, s * hi.y);
            } else {
                v.x = c0 + 0 < dim ? s * row[c0 + 0] : 0.f;
                v.y = c0 + 1 < dim ? s * row[c0 + 1] : 0.f;
                v.z = c0 + 2 < dim ? s * row[c0 + 2] : 0.f;
                v.w = c0 + 3 < dim ? s * row[c0 + 3] : 0.f;
            }
            *reinterpret_cast<float4*>(dst + at) = v;
        }
        if (total_vecs - i <= stride) break;      // the next index would run past the end (and could wrap)
    }
}

// In-place / unpadded form for a workspace that aliases the input: dst[i] = scale[row(i)] * src[i].
template <class Index>
__global__ __launch_bounds__(256) void scale_rows_flat_kernel(float* __restrict__ dst, const float* __restrict__ src,
                                                              const float* __restrict__ scale,
                                                              const uint32_t* __restrict__ rows, Index total, Index dim)
{
    const Index stride = static_cast<Index>(gridDim.x) * blockDim.x;
    for (Index i = static_cast<Index>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += stride) {
        const Index r = i / dim;
        if (row_wanted(rows, r)) dst[i] = scale[r] * src[i];
        if (total - i <= stride) break;
    }
}

// Same for rows of a multiple of 4 floats and 16-byte aligned buffers: one float4 per thread.
template <class Index>
__global__ __launch_bounds__(256) void scale_rows_flat4_kernel(float4* dst, const float4* src,
                                                               const float* __restrict__ scale,
                                                               const uint32_t* __restrict__ rows, Index total_vecs,
                                                               Index vecs_per_row, unsigned swz_mask)
{
    const Index stride = static_cast<Index>(gridDim.x) * blockDim.x;
    for (Index i = static_cast<Index>(blockIdx.x) * blockDim.x + threadIdx.x; i < total_vecs; i += stride) {
        const Index r = i / vecs_per_row;
        if (row_wanted(rows, r)) {
            const float s = scale[r];
            typedef float nt4 __attribute__((ext_vector_type(4)));
            // read once: a non-temporal load leaves the caches to the table (width 16 at R-MAT 22: call 1.119 -> 1.097 ms;
            // the 8-byte loads of the padded form above lose with it)
            const nt4 t = __builtin_nontemporal_load(reinterpret_cast<const nt4*>(src + i));
            float4 v = make_float4(t.x * s, t.y * s, t.z * s, t.w * s);
            dst[static_cast<size_t>(swizzled_row(static_cast<unsigned>(r), swz_mask)) * vecs_per_row + (i - r * vecs_per_row)] = v;
        }
        if (total_vecs - i <= stride) break;
    }
}

// ---------------------------------------------------------------- kernel
// VW: floats per load of the input (row pitch ld_in, `chunks` vectors per row are read);
// OVW: floats per store of the output (row pitch ld_out, columns < width_out are written).
//
// A wave owns TPW * rounds (at most 64) consecutive groups.  It first loads their descriptions,
// one group per lane, into LDS, then runs `rounds` rounds; round r gives the TPW groups
// r * TPW ... to the TPW teams.  The slots of the wave's groups are one contiguous range, of which a
// window of kStageCap slots is staged in LDS and refilled when a round runs past its end.  When the
// last run of a round is continued by the first group of the next round its partial sum is carried
// in registers instead of being flushed, so a long row costs one flush per wave, not one per group.
//
// A "run" is a maximal stretch of adjacent teams whose groups continue one another (same row,
// adjacent in the original group order).  Only such groups are summed across teams, so that
// has_prev of a run's first group and has_next of its last group tell whether the row has
// groups the wave does not hold: if not, the run is stored plainly, otherwise added atomically.
template <int VW, int OVW, int TS, int CPL, int U, bool kPrescaled, class Groups>
__global__ __launch_bounds__(kAggBlock) void aggregate_kernel(
    float* __restrict__ out, const float* __restrict__ in, const int* __restrict__ col,
    const float* __restrict__ scale, Groups groups, int num_parts, int rounds, int chunks, int ld_in, int width_out,
    int ld_out, unsigned swz_mask)
{
    constexpr int TPW = kWave / TS;                  // teams (= groups) per wave and round
    constexpr int kPasses = kStageCap / kWave;       // load instructions per staging pass
    using V = Vec<VW>;
    __shared__ int stage_col[kAggWaves][kStageWords];
    __shared__ float stage_scale[kAggWaves][kPrescaled ? 1 : kStageWords];
    __shared__ int meta_int[kAggWaves][4][kWave];      // first slot, end slot, row, flags of the wave's groups
    __shared__ float meta_scale[kAggWaves][kWave];     // scale of the group's row

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int team = lane / TS;
    const int tl = lane % TS;
    int* my_col = stage_col[wave];
    float* my_scale = stage_scale[wave];
    int* m_beg = meta_int[wave][0];
    int* m_end = meta_int[wave][1];
    int* m_row = meta_int[wave][2];
    int* m_flags = meta_int[wave][3];
    float* m_scale = meta_scale[wave];
    const long long wave_first = (static_cast<long long>(blockIdx.x) * kAggWaves + wave) * TPW * rounds;
    if (wave_first >= num_parts) return;                   // wave-uniform; the LDS rows are wave-private
    // the wave's groups (TPW * rounds <= 64 of them): one group per lane loads its description once,
    // so that the rounds below start from LDS instead of from a chain of dependent global loads
    const int ng = static_cast<int>(min(static_cast<long long>(TPW) * rounds, num_parts - wave_first));
    {
        int gb = 0, ge = 0, rw = 0, fl = 0;
        float sr = 0.f;
        if (lane < ng) {
            const int p = static_cast<int>(wave_first) + lane;
            gb = groups.part_ptr[p];
            ge = groups.part_ptr[p + 1];
            if (ge > gb) {
                rw = groups.row_of(p, gb);
                const bool prev = groups.has_prev(p, rw, gb);
                const bool next = groups.has_next(p, rw, ge, num_parts);
                fl = 16 | (prev ? 1 : 0) | (next ? 2 : 0) | (groups.joins_left(p, prev) ? 4 : 0) |
                     (groups.joins_right(p, next) ? 8 : 0);
                sr = scale[rw];
            }
        }
        m_beg[lane] = gb;
        m_end[lane] = ge;
        m_row[lane] = rw;
        m_flags[lane] = fl;
        m_scale[lane] = sr;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int slots_end = m_end[ng - 1];                   // end of the slot range of the wave's groups
    int win_beg = 0, win_end = 0;                          // staged window [win_beg, win_end), wave-uniform

    V carry[CPL];                // partial sum of the run that continues from the previous round (team 0)
    bool carry_valid = false;    // wave-uniform
    bool carry_outside = false;  // the carried run's row has groups before the run
    int carry_row = 0;
#pragma unroll
    for (int k = 0; k < CPL; ++k)
#pragma unroll
        for (int j = 0; j < VW; ++j) carry[k].v[j] = 0.f;

    for (int round = 0; round < rounds; ++round) {
        const int g0 = round * TPW;
        if (g0 >= ng) break;                                 // wave-uniform
        const int np = min(TPW, ng - g0);
        const bool active = team < np;
        const bool more_rounds = round + 1 < rounds && g0 + TPW < ng;

        int gbeg = 0, gend = 0, row = 0, flags = 0;
        float s_row = 0.f;
        if (active) {
            gbeg = m_beg[g0 + team];
            gend = m_end[g0 + team];
            row = m_row[g0 + team];
            flags = m_flags[g0 + team];
            s_row = m_scale[g0 + team];
        }
        bool live = active && (flags & 16) != 0;
        const int wbeg = m_beg[g0];
        const int wend = m_end[g0 + np - 1];

        V acc[CPL];
#pragma unroll
        for (int k = 0; k < CPL; ++k)
#pragma unroll
            for (int j = 0; j < VW; ++j) acc[k].v[j] = 0.f;

        // the groups of the wave cover one contiguous slot range; a window of it is staged in LDS with
        // coalesced loads and lasts for as many rounds as it covers
        for (int cb = wbeg; cb < wend;) {
            if (cb < win_beg || cb >= win_end) {                 // wave-uniform
                __builtin_amdgcn_wave_barrier();                 // all teams are done with the old window
                const int cn_new = min(kStageCap, slots_end - cb);
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    int c[kPasses / 2];
#pragma unroll
                    for (int r = 0; r < kPasses / 2; ++r) {
                        const int i = lane + (half * (kPasses / 2) + r) * kWave;
                        c[r] = i < cn_new ? __builtin_nontemporal_load(col + cb + i) : 0;   // streamed once: keep it out of the rows' way
                    }
                    if constexpr (!kPrescaled) {
                        float sc[kPasses / 2];
#pragma unroll
                        for (int r = 0; r < kPasses / 2; ++r) {
                            const int i = lane + (half * (kPasses / 2) + r) * kWave;
                            sc[r] = i < cn_new ? scale[c[r] & kStreamIdMask] : 0.f;
                        }
#pragma unroll
                        for (int r = 0; r < kPasses / 2; ++r) {
                            const int i = lane + (half * (kPasses / 2) + r) * kWave;
                            if (i < cn_new) my_scale[stage_index(i)] = sc[r];
                        }
                    }
#pragma unroll
                    for (int r = 0; r < kPasses / 2; ++r) {
                        const int i = lane + (half * (kPasses / 2) + r) * kWave;
                        if (i < cn_new) my_col[stage_index(i)] = c[r];
                    }
                }
                win_beg = cb;
                win_end = cb + cn_new;
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            }
            const int pass_end = min(wend, win_end);

            // every team walks the part of its group that lies in this pass, U rows in flight
            const int lo = max(gbeg, cb);
            const int hi = live ? min(gend, pass_end) : lo;
            for (int i = lo; i < hi; i += U) {
                V v[U][CPL];
                float w[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const bool ok = i + u < hi;
                    const int word = stage_index(ok ? i + u - win_beg : 0);
                    const int c = my_col[word] & kStreamIdMask;     // a plan's ids carry a flag in bit 31
                    if constexpr (!kPrescaled) w[u] = ok ? s_row * my_scale[word] : 0.f;
                    // a separate pre-scaled table holds its rows in swizzled order (mask 0: vertex order)
                    const float* src = in + static_cast<size_t>(kPrescaled ? swizzled_row(c, swz_mask) : c) * ld_in;
#pragma unroll
                    for (int k = 0; k < CPL; ++k) {
                        const int ch = tl + k * TS;
                        if (ok && ch < chunks) {
                            v[u][k] = V::load(src + ch * VW);
                        } else {
#pragma unroll
                            for (int j = 0; j < VW; ++j) v[u][k].v[j] = 0.f;
                        }
                    }
                }
#pragma unroll
                for (int u = 0; u < U; ++u)
#pragma unroll
                    for (int k = 0; k < CPL; ++k)
#pragma unroll
                        for (int j = 0; j < VW; ++j) {
                            if constexpr (kPrescaled) acc[k].v[j] += v[u][k].v[j];
                            else acc[k].v[j] = fmaf(w[u], v[u][k].v[j], acc[k].v[j]);
                        }
            }
            cb = pass_end;
        }
        if constexpr (kPrescaled) {
#pragma unroll
            for (int k = 0; k < CPL; ++k)
#pragma unroll
                for (int j = 0; j < VW; ++j) acc[k].v[j] *= s_row;
        }

        // ---- a round of complete rows (every group is all of its row, nothing carried in): each team
        // stores its sum and the run bookkeeping below is skipped.  Plans order single-group rows next to
        // each other, so on graphs of low degree most rounds take this path.
        if (!carry_valid && __all(!active || (flags & 15) == 0)) {
            if (live) {
                float* dst = out + static_cast<size_t>(row) * ld_out;
#pragma unroll
                for (int k = 0; k < CPL; ++k) {
                    const int c0 = (tl + k * TS) * VW;
#pragma unroll
                    for (int piece = 0; piece < VW / OVW; ++piece) {
                        const int c = c0 + piece * OVW;
                        if (c < width_out) {
                            Vec<OVW> o;
#pragma unroll
                            for (int j = 0; j < OVW; ++j) o.v[j] = acc[k].v[piece * OVW + j];
                            o.store(dst + c);
                        }
                    }
                }
            }
            continue;
        }

        // ---- combine with the carried run, reduce across teams, flush or carry on
        bool prev = live && (flags & 1) != 0;
        const bool next = live && (flags & 2) != 0;
        const bool joins_left = live && (flags & 4) != 0;
        const bool joins_right = live && (flags & 8) != 0;
        bool orphan = false;           // a carried sum met an empty group (malformed input): never store plainly
        if (carry_valid && team == 0) {
            // the first group of this round continues the carried run
            if (!live) { live = true; row = carry_row; orphan = true; }
#pragma unroll
            for (int k = 0; k < CPL; ++k)
#pragma unroll
                for (int j = 0; j < VW; ++j) acc[k].v[j] += carry[k].v[j];
            prev = carry_outside;          // what lies before the carried part, not before this group
        }
        bool head = live;              // this team writes its (possibly combined) sum
        // flags of the run's last group: bit0 the row has groups after it, bit1 the next group continues it
        int tail = ((next || orphan) ? 1 : 0) | (joins_right ? 2 : 0);
        if constexpr (TPW > 1) {
            // a team starts a run unless it continues its (live) left neighbour
            const int live_up = __shfl_up(static_cast<int>(live), TS, kWave);
            const bool starts = !(team > 0 && joins_left && live_up != 0);
            const uint64_t start_lanes = __ballot(starts && tl == 0 && active);
            if (np > 1 && start_lanes == 1ull && __all(!active || live)) {
                // the whole round is one run: butterfly over the teams with DPP / swizzle
#pragma unroll
                for (int k = 0; k < CPL; ++k)
#pragma unroll
                    for (int j = 0; j < VW; ++j) acc[k].v[j] = cross_team_sum<TS>(acc[k].v[j]);
                head = team == 0;
                prev = __shfl(static_cast<int>(prev), 0, kWave) != 0;
                tail = __shfl(tail, (np - 1) * TS, kWave);
            } else if (__any(live && !starts)) {
                // several runs: segmented reduction towards the first team of every run; the flags of
                // the run's last team travel towards the head with the sums
                const uint64_t upto = (lane | (TS - 1)) == 63 ? ~0ull : ((2ull << (lane | (TS - 1))) - 1ull);
                const int key = live ? __popcll(start_lanes & upto) : -1 - team;   // run number, monotone
#pragma unroll
                for (int d = 1; d < TPW; d <<= 1) {
                    const int other = __shfl_down(key, d * TS, kWave);
                    const int other_tail = __shfl_down(tail, d * TS, kWave);
                    const bool take = team + d < TPW && other == key;
                    if (take) tail = other_tail;
#pragma unroll
                    for (int k = 0; k < CPL; ++k)
#pragma unroll
                        for (int j = 0; j < VW; ++j) {
                            const float o = __shfl_down(acc[k].v[j], d * TS, kWave);
                            if (take) acc[k].v[j] += o;
                        }
                }
                head = live && starts;
            }
        }
        // the last run of the round is carried into the next round when the next group continues it
        carry_valid = false;
        if (more_rounds) {
            const uint64_t heads = __ballot(head && tl == 0);
            const int last_team_lane = (np - 1) * TS;
            if (heads && __shfl(static_cast<int>(live), last_team_lane, kWave) != 0) {
                const int h = 63 - __builtin_clzll(heads);           // first lane of the last head team
                // runs are contiguous, so the last head's run ends at the round's last team
                if ((__shfl(tail, h, kWave) & 2) != 0) {
                    carry_valid = true;
                    carry_outside = __shfl(static_cast<int>(prev), h, kWave) != 0;
                    carry_row = __shfl(row, h, kWave);
#pragma unroll
                    for (int k = 0; k < CPL; ++k)
#pragma unroll
                        for (int j = 0; j < VW; ++j) carry[k].v[j] = __shfl(acc[k].v[j], h + tl, kWave);
                    if (lane >= h && lane < h + TS) head = false;    // carried, not flushed
                }
            }
        }
        if (head) {
            const bool outside = prev || (tail & 1) != 0;   // the row also has groups this wave does not hold
            float* dst = out + static_cast<size_t>(row) * ld_out;
#pragma unroll
            for (int k = 0; k < CPL; ++k) {
                const int c0 = (tl + k * TS) * VW;
#pragma unroll
                for (int piece = 0; piece < VW / OVW; ++piece) {
                    const int c = c0 + piece * OVW;
                    if (c < width_out) {      // width_out is a multiple of OVW: a piece is all in or all out
                        if (outside) {
#pragma unroll
                            for (int j = 0; j < OVW; ++j) unsafeAtomicAdd(dst + c + j, acc[k].v[piece * OVW + j]);
                        } else {
                            Vec<OVW> o;
#pragma unroll
                            for (int j = 0; j < OVW; ++j) o.v[j] = acc[k].v[piece * OVW + j];
                            o.store(dst + c);
                        }
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------- dispatch
struct AggTuning {            // process-wide knobs (tuning header)
    std::atomic<int> force_team{0};      // 0 = automatic; otherwise lanes per team (power of two, 4..64)
    std::atomic<int> force_rounds{0};    // 0 = automatic; otherwise rounds per wave
};
static AggTuning g_tuning;
void set_agg_force_team(int ts) { g_tuning.force_team.store(ts); }
void set_agg_force_rounds(int r) { g_tuning.force_rounds.store(r); }
constexpr int kEdgesPerWave = 800;
constexpr int kGroupsPerWave = 64;
constexpr int kMinWaves = 256 * 24 * 4;
constexpr int kMaxRounds = 64;

struct AggShape {
    int group_size;  // the caller's group size (upper bound of a group's length)
    int chunks;      // input vectors read per row
    int ld_in;       // input row pitch (floats)
    int width_out;   // output columns written
    int ld_out;      // output row pitch (floats)
    unsigned swz_mask;   // kRowSwizzleMask when the input is a separate pre-scaled table, else 0
};

template <int VW, int OVW, int TS, int CPL, int U, bool kPrescaled, class Groups>
static hipError_t launch_one(float* out, const float* in, const int* col, const float* scale, Groups g,
                             int num_parts, AggShape sh, hipStream_t stream)
{
    constexpr int TPW = kWave / TS;
    // rounds per wave: at least kEdgesPerWave gathered rows per wave, judged by the caller's
    // group size (an upper bound of the real group length), and at least kGroupsPerWave groups
    // when a round holds fewer than 16 (measured at R-MAT scale 22 with execution plans: width 16, 16
    // groups a round, 1 / 2 / 4 / 8 rounds -> 1.36 / 1.32 / 1.35 / 1.45 ms; width 22, 8 groups a round, gains 9 % from 8 rounds
    // because a long row is then flushed once per 64 groups instead of once per 8)
    int rounds = g_tuning.force_rounds.load();
    if (rounds <= 0) {
        const int per_round = TPW * (sh.group_size > 0 ? sh.group_size : 1);
        rounds = (kEdgesPerWave + per_round - 1) / per_round;
        if (TPW < 16 && rounds < kGroupsPerWave / TPW) rounds = kGroupsPerWave / TPW;
        // small launches keep enough waves to fill the 256 CUs several times over
        const long long fill = num_parts / (static_cast<long long>(TPW) * kMinWaves);
        if (rounds > fill) rounds = static_cast<int>(fill);
    }
    if (rounds < 1) rounds = 1;
    if (rounds > kMaxRounds) rounds = kMaxRounds;
    if (rounds > kWave / TPW) rounds = kWave / TPW;      // a wave describes its groups one per lane
    const long long groups_per_block = static_cast<long long>(TPW) * kAggWaves * rounds;
    const long long grid = (num_parts + groups_per_block - 1) / groups_per_block;
    hipLaunchKernelGGL((aggregate_kernel<VW, OVW, TS, CPL, U, kPrescaled, Groups>),
                       dim3(static_cast<unsigned>(grid)), dim3(kAggBlock), 0, stream, out, in, col, scale, g,
                       num_parts, rounds, sh.chunks, sh.ld_in, sh.width_out, sh.ld_out, sh.swz_mask);
    return hipGetLastError();
}

// One column slab of at most 64*4 input vectors of VW floats.
template <int VW, int OVW, bool kPrescaled, class Groups>
static hipError_t launch_slab(float* out, const float* in, const int* col, const float* scale, Groups g,
                              int num_parts, AggShape sh, hipStream_t stream)
{
    const int chunks = sh.chunks;
    int ts = 4;
    while (ts < 64 && ts < chunks) ts <<= 1;
    const int ft = g_tuning.force_team.load();
    if (ft >= 4 && ft <= 64 && (ft & (ft - 1)) == 0 && chunks <= ft) ts = ft;   // only wider teams can be forced
    const int cpl = (chunks + ts - 1) / ts;
#define EPPGCN_LAUNCH(TS_, CPL_, U_) \
    return launch_one<VW, OVW, TS_, CPL_, U_, kPrescaled, Groups>(out, in, col, scale, g, num_parts, sh, stream)
    if (cpl <= 1) {
        switch (ts) {
            case 4: EPPGCN_LAUNCH(4, 1, 8);
            case 8: EPPGCN_LAUNCH(8, 1, 8);
            case 16: EPPGCN_LAUNCH(16, 1, 8);
            case 32: EPPGCN_LAUNCH(32, 1, 8);
            default: EPPGCN_LAUNCH(64, 1, 8);
        }
    } else if (cpl == 2) {
        EPPGCN_LAUNCH(64, 2, 4);
    } else {
        EPPGCN_LAUNCH(64, 4, 2);
    }
#undef EPPGCN_LAUNCH
}

template <int VW, int OVW, class Groups>
static hipError_t slab_either(bool prescaled, float* out, const float* in, const int* col, const float* scale,
                              Groups g, int num_parts, AggShape sh, hipStream_t stream)
{
    if (prescaled) return launch_slab<VW, OVW, true>(out, in, col, scale, g, num_parts, sh, stream);
    return launch_slab<VW, OVW, false>(out, in, col, scale, g, num_parts, sh, stream);
}

// Row pitch of the pre-scaled workspace: rows of up to 128 bytes are padded to a power of two
// (16 / 32 / 64 / 128 bytes) so that a row never straddles a 128-byte cache line; wider rows to
// whole 32-byte sectors.  Measured at width 22 (88-byte rows): pitch 24 floats 2.06 ms, pitch 32
// floats 1.91 ms per forward launch, although the table grows by a third.
int workspace_pitch(int dim)
{
    if (dim <= 4) return 4;
    if (dim <= 8) return 8;
    if (dim <= 16) return 16;
    if (dim <= 32) return 32;
    return (dim + 7) / 8 * 8;
}

// a separate table holds its rows in swizzled order, whole blocks of 4096 rows
size_t feature_workspace_floats(long long num_nodes, int dim)
{
    return static_cast<size_t>(swizzle_padded_rows(num_nodes)) * static_cast<size_t>(workspace_pitch(dim));
}

// Restricted form of the pass for a sparse row set: a wave looks at 64 rows at a time, collects those
// whose bit is set and scales them one 16-byte vector per lane, so the cost follows the rows that are
// gathered instead of the size of the matrix.  dst rows are ld_dst floats apart (a multiple of 4,
// 16-byte aligned); dst may be src (then ld_dst == dim).
__global__ __launch_bounds__(256) void scale_listed_rows_kernel(float* __restrict__ dst, const float* __restrict__ src,
                                                                const float* __restrict__ scale,
                                                                const uint32_t* __restrict__ rows, unsigned num_rows,
                                                                unsigned vecs_per_row, unsigned dim, bool pairs,
                                                                bool quads, unsigned swz_mask)
{
    __shared__ int lists[4][kWave];
    int* list = lists[threadIdx.x / kWave];
    const unsigned lane = threadIdx.x & (kWave - 1);
    const unsigned waves = gridDim.x * 4u;
    const unsigned blocks64 = (num_rows + 63u) / 64u;
    for (unsigned b = blockIdx.x * 4u + threadIdx.x / kWave; b < blocks64; b += waves) {
        const unsigned r0 = b * 64u + lane;
        const bool wanted = r0 < num_rows && ((rows[r0 >> 5] >> (r0 & 31)) & 1u) != 0;
        const unsigned count = compact_wanted_rows(list, r0, wanted);
        const unsigned total = count * vecs_per_row;
        for (unsigned t = lane; t < total; t += kWave) {
            const unsigned k = t / vecs_per_row;
            const unsigned c0 = (t - k * vecs_per_row) * 4;
            const size_t r = static_cast<size_t>(list[k]);
            const float s = scale[r];
            const float* row = src + r * dim;
            float4 v;
            if (quads) {                 // width a multiple of 4, 16-byte aligned source: whole vectors, read once
                typedef float nt4 __attribute__((ext_vector_type(4)));
                nt4 q = {0.f, 0.f, 0.f, 0.f};
                if (c0 < dim) q = __builtin_nontemporal_load(reinterpret_cast<const nt4*>(row + c0));
                v = make_float4(s * q.x, s * q.y, s * q.z, s * q.w);
            } else if (pairs) {
                const float2 lo = c0 < dim ? *reinterpret_cast<const float2*>(row + c0) : make_float2(0.f, 0.f);
                const float2 hi = c0 + 2 < dim ? *reinterpret_cast<const float2*>(row + c0 + 2) : make_float2(0.f, 0.f);
                v = make_float4(s * lo.x, s * lo.y, s * hi.x, s * hi.y);
            } else {
                v.x = c0 + 0 < dim ? s * row[c0 + 0] : 0.f;
                v.y = c0 + 1 < dim ? s * row[c0 + 1] : 0.f;
                v.z = c0 + 2 < dim ? s * row[c0 + 2] : 0.f;
                v.w = c0 + 3 < dim ? s * row[c0 + 3] : 0.f;
            }
            *reinterpret_cast<float4*>(dst + static_cast<size_t>(swizzled_row(static_cast<unsigned>(r), swz_mask)) *
                                                 (static_cast<size_t>(vecs_per_row) * 4) + c0) = v;
        }
    }
}

template <class Index>
static void launch_scale_rows_typed(float* dst, const float* src, const float* scale, const uint32_t* rows,
                                    long long num_nodes, int dim, int ld_dst, unsigned swz_mask, hipStream_t stream)
{
    auto grid_for = [](long long threads) {
        long long blocks = (threads + 255) / 256;
        if (blocks > 256 * 32) blocks = 256 * 32;
        return dim3(static_cast<unsigned>(blocks < 1 ? 1 : blocks));
    };
    const bool in_place = dst == src;
    if (in_place || ld_dst == dim) {
        const long long total = num_nodes * dim;
        if (dim % 4 == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0 && reinterpret_cast<uintptr_t>(src) % 16 == 0) {
            hipLaunchKernelGGL((scale_rows_flat4_kernel<Index>), grid_for(total / 4), dim3(256), 0, stream,
                               reinterpret_cast<float4*>(dst), reinterpret_cast<const float4*>(src), scale, rows,
                               static_cast<Index>(total / 4), static_cast<Index>(dim / 4), in_place ? 0u : swz_mask);
            return;
        }
        if (in_place || swz_mask == 0) {
            hipLaunchKernelGGL((scale_rows_flat_kernel<Index>), grid_for(total), dim3(256), 0, stream, dst, src, scale, rows,
                               static_cast<Index>(total), static_cast<Index>(dim));
            return;
        }
        // a separate table without padding whose source is not 16-byte aligned: the general kernel below
    }
    const long long vecs = num_nodes * (ld_dst / 4);
    hipLaunchKernelGGL((scale_rows_kernel<Index>), grid_for(vecs), dim3(256), 0, stream, dst, src, scale, rows,
                       static_cast<Index>(vecs), static_cast<Index>(ld_dst / 4), static_cast<Index>(dim),
                       dim % 2 == 0 && reinterpret_cast<uintptr_t>(src) % 8 == 0, swz_mask);
}

// swz_mask: kRowSwizzleMask for a separate table (rows in swizzled order), 0 for one in vertex order
static int launch_scale_rows(float* dst, const float* src, const float* scale, const uint32_t* rows, int num_nodes,
                             int dim, int ld_dst, unsigned swz_mask, hipStream_t stream)
{
    if (static_cast<long long>(num_nodes) * dim == 0) return kOk;
    if (rows && ld_dst % 4 == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0 && !force_wide_index()) {
        long long blocks = (static_cast<long long>(num_nodes) + 255) / 256;     // one wave per 64 rows
        if (blocks > 256 * 16) blocks = 256 * 16;
        hipLaunchKernelGGL(scale_listed_rows_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, dst, src,
                           scale, rows, static_cast<unsigned>(num_nodes), static_cast<unsigned>(ld_dst / 4),
                           static_cast<unsigned>(dim), dim % 2 == 0 && reinterpret_cast<uintptr_t>(src) % 8 == 0,
                           dim % 4 == 0 && reinterpret_cast<uintptr_t>(src) % 16 == 0 && dst != src,
                           dst == src ? 0u : swz_mask);
        EPPGCN_HIP(hipGetLastError());
        return kOk;
    }
    const long long elems = swizzle_padded_rows(num_nodes) * (ld_dst > dim ? ld_dst : dim);
    if (elems < (1ll << 32) && !force_wide_index()) launch_scale_rows_typed<unsigned>(dst, src, scale, rows, num_nodes, dim, ld_dst, swz_mask, stream);
    else launch_scale_rows_typed<unsigned long long>(dst, src, scale, rows, num_nodes, dim, ld_dst, swz_mask, stream);
    EPPGCN_HIP(hipGetLastError());
    return kOk;
}

static int vector_width(int pitch, int width, const void* p)
{
    const uintptr_t a = reinterpret_cast<uintptr_t>(p);
    if (pitch % 4 == 0 && width % 4 == 0 && a % 16 == 0) return 4;
    if (pitch % 2 == 0 && width % 2 == 0 && a % 8 == 0) return 2;
    return 1;
}

// workspace: nullptr (per-edge scale gather), the input pointer itself (scaled in place, pitch dim)
// or a separate buffer of feature_workspace_floats() floats (padded pitch).
bool stream_covers(int num_nodes, int dim, int ld_in, const float* table);                     // stream.hip
int launch_aggregate_stream(float* out, float* partial, const float* table, const int* scol, const StreamView& sv,
                            const StreamInfo& info, const float* scale, int num_nodes, int dim, int ld_in,
                            hipStream_t stream);

// The stream form of the plan is used when the host knows it (eppgcn_plan_status has read its header), the
// rows are gathered from a separate pre-scaled workspace, the shape fits the stream kernel and the workspace has
// room for the partial sums behind the table.
static bool stream_usable(const StreamInfo* info, const float* in, const float* workspace, size_t workspace_floats,
                          int num_nodes, int dim, int num_parts)
{
    if (!info || !workspace || workspace == in) return false;
    if (!info->header.valid || info->num_parts != num_parts || info->num_nodes != num_nodes) return false;
    const int ld = workspace_pitch(dim);
    if (!stream_covers(num_nodes, dim, ld, workspace)) return false;
    return workspace_floats >= (static_cast<size_t>(swizzle_padded_rows(num_nodes)) + static_cast<size_t>(info->header.num_partials)) * ld;
}

// which kernel family the calling thread's last planned aggregation call ran (1 = stream form)
static thread_local int g_last_used_stream = 0;
int last_call_used_stream() { return g_last_used_stream; }

// written: nullptr, or where the caller wants the bitmap of the rows this call writes (one bit per vertex, inside the
// plan); the rows without any slot are then left as they are instead of being cleared, and *count is their complement.
static int aggregate_stream_call(float* out, const float* in, const int* scol, const float* scale, const StreamInfo& info,
                                 const void* plan, int num_nodes, int dim, float* workspace, hipStream_t stream,
                                 double* sink, double* sink2, const uint32_t* gathered_rows,
                                 const uint32_t** written = nullptr, long long* count = nullptr)
{
    const StreamView sv = stream_view(const_cast<void*>(plan), info.num_parts, info.num_slots, info.num_nodes);
    const int ld = workspace_pitch(dim);
    g_last_used_stream = 1;
    if (written) {
        *written = sv.touched;
        if (count) *count = static_cast<long long>(num_nodes) - info.header.empty_rows;
    }
    // only rows without any slot are left to a clear: every other row is written by the stream kernel or the fix-up
    if (info.header.empty_rows > 0 && !written) {
        KernelTimer timer(stream, phase_sink(0));
        if (2ll * info.header.empty_rows <= num_nodes) {
            if (int rc = launch_zero_rows_unless(out, sv.touched, num_nodes, dim, stream)) return rc;
        } else {
            if (int rc = launch_zero_words(out, static_cast<size_t>(num_nodes) * dim, stream)) return rc;
        }
    }
    if (in) {
        KernelTimer timer(stream, phase_sink(1));
        if (int rc = launch_scale_rows(workspace, in, scale, gathered_rows, num_nodes, dim, ld, kRowSwizzleMask, stream)) return rc;
    }
    KernelTimer timer(stream, sink, sink2);
    return launch_aggregate_stream(out, workspace + static_cast<size_t>(swizzle_padded_rows(num_nodes)) * ld, workspace, scol, sv, info, scale,
                                   num_nodes, dim, ld, stream);
}

template <class Groups>
static int aggregate_dispatch(float* out, const float* in, const int* col, const float* scale, Groups g,
                              int num_nodes, int dim, int num_parts, int group_size, float* workspace,
                              hipStream_t stream, double* sink, double* sink2, const uint32_t* single_rows = nullptr,
                              const uint32_t* gathered_rows = nullptr)
{
    const bool prescaled = workspace != nullptr;
    int ld_in = dim;
    g_last_used_stream = 0;
    // rows the kernel writes with one plain store (a plan knows them) need no clearing; with fewer
    // groups than half the rows most rows have no group at all and the plain fill is the faster clear
    {
        KernelTimer timer(stream, phase_sink(0));
        if (single_rows && 2ll * num_parts >= num_nodes) {
            if (int rc = launch_zero_rows_unless(out, single_rows, num_nodes, dim, stream)) return rc;
        } else {
            if (int rc = launch_zero_words(out, static_cast<size_t>(num_nodes) * dim, stream)) return rc;
        }
    }
    if (num_parts == 0) return kOk;
    // a separate table (not the input scaled in place) holds its rows in swizzled order
    const unsigned swz_mask = (prescaled && workspace != in) ? kRowSwizzleMask : 0u;
    if (prescaled) {
        // in == nullptr: the caller (the dense update) already wrote the scaled, padded rows
        ld_in = workspace == in ? dim : workspace_pitch(dim);
        if (in) {
            KernelTimer timer(stream, phase_sink(1));
            if (int rc = launch_scale_rows(workspace, in, scale, gathered_rows, num_nodes, dim, ld_in, swz_mask, stream)) return rc;
        }
        in = workspace;
    }
    KernelTimer timer(stream, sink, sink2);   // brackets the aggregation kernel alone
    // rows with the caller's pitch are read and written with the same vector width; padded
    // workspace rows are read 16 bytes at a time whatever the output alignment allows
    int ovw_eff = vector_width(dim, dim, out);
    int vw;
    if (ld_in == dim) {
        const int vin = vector_width(dim, dim, in);
        vw = ovw_eff = vin < ovw_eff ? vin : ovw_eff;
    } else {
        vw = vector_width(ld_in, ld_in, in);
        if (vw < ovw_eff) ovw_eff = vw;
    }
    const int slab = 256 * vw;                          // input columns one launch covers
    for (int c0 = 0; c0 < ld_in; c0 += slab) {
        if (c0 >= dim) break;
        AggShape sh;
        sh.group_size = group_size;
        const int in_cols = ld_in - c0 < slab ? ld_in - c0 : slab;
        sh.chunks = in_cols / vw;
        sh.ld_in = ld_in;
        sh.width_out = dim - c0 < slab ? dim - c0 : slab;
        sh.ld_out = dim;
        sh.swz_mask = swz_mask;
        hipError_t e;
#define EPPGCN_SLAB(VW_, OVW_) slab_either<VW_, OVW_>(prescaled, out + c0, in + c0, col, scale, g, num_parts, sh, stream)
        if (vw == 4 && ovw_eff == 4) e = EPPGCN_SLAB(4, 4);
        else if (vw == 4 && ovw_eff == 2) e = EPPGCN_SLAB(4, 2);
        else if (vw == 4) e = EPPGCN_SLAB(4, 1);
        else if (vw == 2 && ovw_eff == 2) e = EPPGCN_SLAB(2, 2);
        else if (vw == 2) e = EPPGCN_SLAB(2, 1);
        else e = EPPGCN_SLAB(1, 1);
#undef EPPGCN_SLAB
        if (e != hipSuccess) return hip_fail(e, "aggregate kernel launch");
    }
    return kOk;
}

// plan: nullptr, or an execution plan built for exactly these groups.
int aggregate_forward_groups(float* out, const float* in, const int* col, const float* scale,
                             const int* part_ptr, const int* part2node, const void* plan, int num_nodes, int dim,
                             int num_parts, int group_size, float* workspace, size_t workspace_floats,
                             hipStream_t stream, double* sink, double* sink2)
{
    if (plan && num_parts > 0) {
        const PlanView v = plan_view(const_cast<void*>(plan), num_parts, num_nodes);
        StreamInfo info;
        if (stream_usable(find_stream_info(plan, &info), in, workspace, workspace_floats, num_nodes, dim, num_parts))
            return aggregate_stream_call(out, in, v.col, scale, info, plan, num_nodes, dim, workspace, stream, sink, sink2,
                                         nullptr);
        return aggregate_dispatch(out, in, v.col, scale, PlanGroups{v.ptr, v.row, v.flags}, num_nodes, dim, num_parts,
                                  group_size, workspace, stream, sink, sink2, v.single);
    }
    return aggregate_dispatch(out, in, col, scale, ForwardGroups{part_ptr, part2node}, num_nodes, dim, num_parts,
                              group_size, workspace, stream, sink, sink2);
}

// gathered_rows: nullptr, or one bit per vertex, set for every vertex that occurs in edge_list; the
// pre-scaling pass then skips the rows no group reads.
int aggregate_compacted_groups(float* out, const float* in, const int* ids, const int* part_ptr,
                               const int* edge_list, const float* scale, const void* plan, int num_nodes, int dim,
                               int num_parts, int group_size, float* workspace, size_t workspace_floats,
                               const uint32_t* gathered_rows, hipStream_t stream, double* sink, double* sink2,
                               const uint32_t** written, long long* num_written)
{
    if (written) *written = nullptr;        // unless the stream form runs, every row of `out` is defined
    if (plan && num_parts > 0) {
        const PlanView v = plan_view(const_cast<void*>(plan), num_parts, num_nodes);
        StreamInfo info;
        if (stream_usable(find_stream_info(plan, &info), in, workspace, workspace_floats, num_nodes, dim, num_parts))
            return aggregate_stream_call(out, in, v.col, scale, info, plan, num_nodes, dim, workspace, stream, sink, sink2,
                                         gathered_rows, written, num_written);
        return aggregate_dispatch(out, in, v.col, scale, PlanGroups{v.ptr, v.row, v.flags}, num_nodes, dim, num_parts,
                                  group_size, workspace, stream, sink, sink2, v.single, gathered_rows);
    }
    return aggregate_dispatch(out, in, edge_list, scale, CompactedGroups{part_ptr, ids}, num_nodes, dim, num_parts,
                              group_size, workspace, stream, sink, sink2, nullptr, gathered_rows);
}

}  // namespace eppgcn
