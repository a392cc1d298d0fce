// Neighbour-group aggregation for gfx950 (wave64): forward SpMM, unpruned
// backward SpMM and the pruned backward that walks the compacted execution path.
//
// Replaces the reference's spmm_forward_cuda_kernel / spmm_backward_cuda_kernel
// (EPPGCN/GCNConv/EPPGCN_kernel.cu:204-295, :471-545) and ours_backward_cuda_kernel
// (:626-670).  Same contract, different machine mapping:
//
//   out[r, :] = sum over the slots e of every group of row r of
//               fl32(s[r] * s[col[e]]) * in[col[e], :]
//
// Mapping.  A wave of 64 lanes is cut into teams of TS lanes; a team owns one
// neighbour group and its lanes stripe the feature row in contiguous vectors of
// VW floats (lane l of the team holds columns [l*VW, l*VW+VW), then +TS*VW ...),
// so one gather instruction fetches 64/TS whole neighbour rows with contiguous
// bytes per row.  The groups of a wave are consecutive, hence their CSR slots are
// one contiguous range: the wave first stages that range coalesced into LDS as
// (column id, neighbour scale) pairs, which turns the per-neighbour dependent
// chain "id -> scale -> row" into three batched phases with many requests in
// flight.  Partial sums live in registers.  Flush: a row whose groups all sit in
// this wave is reduced across teams with DPP / ds_swizzle and written with plain
// stores; a row with a single group is stored directly; only rows spread over
// several waves use float atomics.
#include "common.hpp"

namespace eppgcn {

constexpr int kAggBlock = 256;
constexpr int kAggWaves = kAggBlock / kWave;
constexpr int kStageCap = 512;   // staged (column, scale) pairs per wave and pass

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
    __device__ void store(float* p) const { *reinterpret_cast<float2*>(p) = make_float2(v[0], v[1]); }
};
template <> struct Vec<4> {
    float v[4];
    __device__ static Vec load(const float* p)
    {
        float4 t = *reinterpret_cast<const float4*>(p);
        Vec r; r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z; r.v[3] = t.w; return r;
    }
    __device__ void store(float* p) const { *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]); }
};

// ---------------------------------------------------------------- group sources
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
};

// ---------------------------------------------------------------- kernel
template <int VW, int TS, int CPL, int U, class Groups>
__global__ __launch_bounds__(kAggBlock) void aggregate_kernel(
    float* __restrict__ out, const float* __restrict__ in, const int* __restrict__ col,
    const float* __restrict__ scale, Groups groups, int num_parts, int width, int ld)
{
    constexpr int TPW = kWave / TS;      // teams (= groups) per wave
    using V = Vec<VW>;
    __shared__ int2 stage[kAggWaves][kStageCap];

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int team = lane / TS;
    const int tl = lane % TS;
    const long long p0 = (static_cast<long long>(blockIdx.x) * kAggWaves + wave) * TPW;
    if (p0 >= num_parts) return;                         // wave-uniform
    const int np = min(TPW, static_cast<int>(num_parts - p0));
    const int p = static_cast<int>(p0) + team;
    const bool active = team < np;
    const int chunks = width / VW;                       // vectors per feature row

    int gbeg = 0, gend = 0, row = 0;
    float s_row = 0.f;
    if (active) {
        gbeg = groups.part_ptr[p];
        gend = groups.part_ptr[p + 1];
        if (gend > gbeg) {
            row = groups.row_of(p, gbeg);
            s_row = scale[row];
        }
    }
    const bool live = active && gend > gbeg;
    const int wbeg = __shfl(gbeg, 0, kWave);
    const int wend = __shfl(gend, (np - 1) * TS, kWave);

    V acc[CPL];
#pragma unroll
    for (int k = 0; k < CPL; ++k)
#pragma unroll
        for (int j = 0; j < VW; ++j) acc[k].v[j] = 0.f;

    int2* my_stage = stage[wave];
    for (int cb = wbeg; cb < wend; cb += kStageCap) {
        const int cn = min(kStageCap, wend - cb);
        // phase 1+2: coalesced column ids, then one scale gather per staged slot
        {
            int c[kStageCap / kWave];
            float sc[kStageCap / kWave];
#pragma unroll
            for (int r = 0; r < kStageCap / kWave; ++r) {
                const int i = lane + r * kWave;
                c[r] = i < cn ? col[cb + i] : 0;
            }
#pragma unroll
            for (int r = 0; r < kStageCap / kWave; ++r) {
                const int i = lane + r * kWave;
                sc[r] = i < cn ? scale[c[r]] : 0.f;
            }
#pragma unroll
            for (int r = 0; r < kStageCap / kWave; ++r) {
                const int i = lane + r * kWave;
                if (i < cn) my_stage[i] = make_int2(c[r], __float_as_int(sc[r]));
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        // phase 3: every team walks the part of its group that lies in this pass
        const int lo = max(gbeg, cb);
        const int hi = live ? min(gend, cb + cn) : lo;
        for (int i = lo; i < hi; i += U) {
            V v[U][CPL];
            float w[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const bool ok = i + u < hi;
                const int2 st = my_stage[ok ? i + u - cb : 0];
                w[u] = ok ? s_row * __int_as_float(st.y) : 0.f;
                const float* src = in + static_cast<size_t>(st.x) * ld;
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
                    for (int j = 0; j < VW; ++j) acc[k].v[j] = fmaf(w[u], v[u][k].v[j], acc[k].v[j]);
        }
        __builtin_amdgcn_wave_barrier();   // all teams are done with the stage before it is refilled
    }

    // ---- flush
    const bool prev = live && groups.has_prev(p, row, gbeg);
    const bool next = live && groups.has_next(p, row, gend, num_parts);
    if constexpr (TPW > 1) {
        const int row0 = __shfl(row, 0, kWave);
        const bool one_row = np > 1 && __all(!active || (live && row == row0));
        if (one_row) {
            // every group of this wave belongs to one row: reduce across teams in registers
#pragma unroll
            for (int k = 0; k < CPL; ++k)
#pragma unroll
                for (int j = 0; j < VW; ++j) acc[k].v[j] = cross_team_sum<TS>(acc[k].v[j]);
            const bool outside = __shfl(static_cast<int>(prev), 0, kWave) ||
                                 __shfl(static_cast<int>(next), (np - 1) * TS, kWave);
            if (team == 0) {
                float* dst = out + static_cast<size_t>(row0) * ld;
#pragma unroll
                for (int k = 0; k < CPL; ++k) {
                    const int ch = tl + k * TS;
                    if (ch < chunks) {
                        if (outside) {
#pragma unroll
                            for (int j = 0; j < VW; ++j) unsafeAtomicAdd(dst + ch * VW + j, acc[k].v[j]);
                        } else {
                            acc[k].store(dst + ch * VW);
                        }
                    }
                }
            }
            return;
        }
    }
    if (live) {
        float* dst = out + static_cast<size_t>(row) * ld;
#pragma unroll
        for (int k = 0; k < CPL; ++k) {
            const int ch = tl + k * TS;
            if (ch < chunks) {
                if (prev || next) {
#pragma unroll
                    for (int j = 0; j < VW; ++j) unsafeAtomicAdd(dst + ch * VW + j, acc[k].v[j]);
                } else {
                    acc[k].store(dst + ch * VW);
                }
            }
        }
    }
}

// ---------------------------------------------------------------- dispatch
struct AggTuning {
    int force_team = 0;      // 0 = automatic; otherwise lanes per team (power of two, 4..64)
};
static AggTuning g_tuning;
void set_agg_force_team(int ts) { g_tuning.force_team = ts; }

template <int VW, int TS, int CPL, int U, class Groups>
static hipError_t launch_one(float* out, const float* in, const int* col, const float* scale, Groups g,
                             int num_parts, int width, int ld, hipStream_t stream)
{
    constexpr int TPW = kWave / TS;
    const long long groups_per_block = static_cast<long long>(TPW) * kAggWaves;
    const long long grid = (num_parts + groups_per_block - 1) / groups_per_block;
    hipLaunchKernelGGL((aggregate_kernel<VW, TS, CPL, U, Groups>), dim3(static_cast<unsigned>(grid)),
                       dim3(kAggBlock), 0, stream, out, in, col, scale, g, num_parts, width, ld);
    return hipGetLastError();
}

// One column slab of at most 64*4 vectors of VW floats.
template <int VW, class Groups>
static hipError_t launch_slab(float* out, const float* in, const int* col, const float* scale, Groups g,
                              int num_parts, int width, int ld, hipStream_t stream)
{
    const int chunks = width / VW;
    int ts = 4;
    while (ts < 64 && ts < chunks) ts <<= 1;
    if (g_tuning.force_team >= 4 && g_tuning.force_team <= 64 &&
        (g_tuning.force_team & (g_tuning.force_team - 1)) == 0 && chunks <= 4 * g_tuning.force_team &&
        (g_tuning.force_team == 64 || chunks <= 2 * g_tuning.force_team))
        ts = g_tuning.force_team;
    const int cpl = (chunks + ts - 1) / ts;
#define EPPGCN_LAUNCH(TS_, CPL_, U_) \
    return launch_one<VW, TS_, CPL_, U_, Groups>(out, in, col, scale, g, num_parts, width, ld, stream)
    if (cpl <= 1) {
        switch (ts) {
            case 4: EPPGCN_LAUNCH(4, 1, 8);
            case 8: EPPGCN_LAUNCH(8, 1, 8);
            case 16: EPPGCN_LAUNCH(16, 1, 8);
            case 32: EPPGCN_LAUNCH(32, 1, 8);
            default: EPPGCN_LAUNCH(64, 1, 8);
        }
    } else if (cpl == 2) {
        switch (ts) {
            case 4: EPPGCN_LAUNCH(4, 2, 4);
            case 8: EPPGCN_LAUNCH(8, 2, 4);
            case 16: EPPGCN_LAUNCH(16, 2, 4);
            case 32: EPPGCN_LAUNCH(32, 2, 4);
            default: EPPGCN_LAUNCH(64, 2, 4);
        }
    } else {
        EPPGCN_LAUNCH(64, 4, 2);
    }
#undef EPPGCN_LAUNCH
}

template <class Groups>
static int aggregate_dispatch(float* out, const float* in, const int* col, const float* scale, Groups g,
                              int num_nodes, int dim, int num_parts, hipStream_t stream, double* sink, double* sink2)
{
    EPPGCN_HIP(hipMemsetAsync(out, 0, static_cast<size_t>(num_nodes) * dim * sizeof(float), stream));
    if (num_parts == 0) return kOk;
    KernelTimer timer(stream, sink, sink2);   // brackets the aggregation kernel(s) only, not the clear
    const uintptr_t bits = reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(in);
    int vw = 1;
    if (dim % 4 == 0 && bits % 16 == 0) vw = 4;
    else if (dim % 2 == 0 && bits % 8 == 0) vw = 2;
    const int slab = 256 * vw;                          // columns one launch covers
    for (int c0 = 0; c0 < dim; c0 += slab) {
        const int width = dim - c0 < slab ? dim - c0 : slab;
        hipError_t e;
        if (vw == 4) e = launch_slab<4>(out + c0, in + c0, col, scale, g, num_parts, width, dim, stream);
        else if (vw == 2) e = launch_slab<2>(out + c0, in + c0, col, scale, g, num_parts, width, dim, stream);
        else e = launch_slab<1>(out + c0, in + c0, col, scale, g, num_parts, width, dim, stream);
        if (e != hipSuccess) return hip_fail(e, "aggregate kernel launch");
    }
    return kOk;
}

int aggregate_forward_groups(float* out, const float* in, const int* col, const float* scale,
                             const int* part_ptr, const int* part2node, int num_nodes, int dim,
                             int num_parts, hipStream_t stream, double* sink, double* sink2)
{
    return aggregate_dispatch(out, in, col, scale, ForwardGroups{part_ptr, part2node}, num_nodes, dim,
                              num_parts, stream, sink, sink2);
}

int aggregate_compacted_groups(float* out, const float* in, const int* ids, const int* part_ptr,
                               const int* edge_list, const float* scale, int num_nodes, int dim,
                               int num_parts, hipStream_t stream, double* sink, double* sink2)
{
    return aggregate_dispatch(out, in, edge_list, scale, CompactedGroups{part_ptr, ids}, num_nodes, dim,
                              num_parts, stream, sink, sink2);
}

}  // namespace eppgcn
