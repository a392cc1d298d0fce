// Dense update of a GCN layer: the three matrix products the reference computes with torch::mm
// around the aggregation (EPPGCN/GCNConv/EPPGCN_kernel.cu:142 X*W, :614 dX = G*W^T,
// :615 dW = X^T*G), written for tall-and-skinny shapes (millions of rows, tens of columns)
// where the work is bound by streaming the tall operand from HBM once.
//
// All three run on the fp32 matrix cores with v_mfma_f32_16x16x4_f32 (one wave computes a
// 16x16 tile of C += A[16x4] * B[4x16]; lane l supplies A[l%16][l/16] and B[l/16][l%16] and
// holds C[4*(l/16) + v][l%16] in accumulator register v).  The rows and weight kernels read the tall
// operand straight from global memory in the operand layout, without staging through LDS:
//
//   rows kernel    out[r, m] = f(r, m) * sum_k act(X[r, k]) * Wop(k, m)      (X*W and G*W^T)
//                  tile: 16 output columns (MFMA rows) x 16 matrix rows (MFMA columns); a lane
//                  reads VW consecutive floats of "its" row per step, the small operand sits in
//                  LDS in operand order; epilogues fuse the per-row scale of the aggregation
//                  weights, the zero padding of the pre-scaled feature table, the ReLU of the
//                  layer input and the ReLU mask of the gradient.
//   weight kernel  dW[k, d] = sum_r act(X[r, k]) * G[r, d]
//                  tile: 16 k x 16 d, reduction over 4 rows per instruction; every wave owns a
//                  contiguous range of rows, block partial sums go to a workspace and a second
//                  kernel adds them in a fixed order (deterministic, no float atomics).
//   backward kernel  both gradients of a narrow layer (<= 16 inputs, <= 32 gradient columns) in one pass:
//                  the 16 rows of a step are copied to LDS with full 16-byte loads and both products take
//                  their operands from there, accumulated exactly as the two kernels above do it.
//
// Row bitmap (the backward products of a pruned layer; the reference sketches the same with an index,
// `torch::mm(X.index({mask}).transpose(0,1), d_input_prime.index({mask}))`, EPPGCN_kernel.cu:607,616): with `rows`
// given, a row of the tall operands whose bit is clear is taken as zero and never read - neither the gradient
// row, which then need not hold defined values, nor the layer-input row that would be multiplied with it.
#include "common.hpp"

namespace eppgcn {

typedef float floatx4 __attribute__((ext_vector_type(4)));

// bits of the 16 rows from r0 on (r0 a multiple of 16); all set without a bitmap
__device__ __forceinline__ unsigned tile_row_bits(const uint32_t* __restrict__ rows, long long r0)
{
    return rows ? (rows[r0 >> 5] >> (r0 & 31)) & 0xffffu : 0xffffu;
}

constexpr int kUpdateThreads = 256;
constexpr int kUpdateWaves = kUpdateThreads / kWave;
constexpr int kTileRows = 16;
constexpr int kMaxWeightBlocks = 1024;
constexpr size_t kMaxOperandLds = 64 * 1024;

__device__ __forceinline__ floatx4 mfma16(float a, float b, floatx4 c)
{
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

// ---------------------------------------------------------------- rows kernel
// Reduction index of lane (i = l%16, j = l/16), step t, component v:  k = (4*t + j)*VW + v.
// Any assignment of k to (step, slot) is valid as long as both operands use the same one; this
// one lets a lane fetch VW consecutive floats of its row with one load.
template <int VW>
__device__ __forceinline__ void load_row_piece(float (&x)[VW], const float* __restrict__ row, int k, int K,
                                               bool relu)
{
    if (k + VW <= K) {
        if constexpr (VW == 4) {
            const float4 t = *reinterpret_cast<const float4*>(row + k);
            x[0] = t.x; x[1] = t.y; x[2] = t.z; x[3] = t.w;
        } else if constexpr (VW == 2) {
            const float2 t = *reinterpret_cast<const float2*>(row + k);
            x[0] = t.x; x[1] = t.y;
        } else {
            x[0] = row[k];
        }
    } else {
#pragma unroll
        for (int v = 0; v < VW; ++v) x[v] = k + v < K ? row[k + v] : 0.f;
    }
    if (relu) {
#pragma unroll
        for (int v = 0; v < VW; ++v) x[v] = fmaxf(x[v], 0.f);
    }
}

struct RowsArgs {
    float* out;              // [N, ld_out]; columns [0, out_cols) are written, [M, out_cols) with zeros
    const float* x;          // [N, ld_x], K valid columns
    const float* w;          // small operand: element (k, m) at w[k*sk + m*sm]
    const float* scale;      // per-row factor or nullptr
    const float* relu_ref;   // [N, ld_ref] or nullptr: out[r, m] is zeroed where relu_ref[r, m] <= 0
    long long n;
    long long sk, sm;
    int ld_out, out_cols, ld_x, ld_ref;
    int K, M;
    int relu_in;             // apply max(x, 0) to X on load
    int vec_store;           // 0: scalar stores; 1: rows of out are 16-byte aligned; 2: the same, non-temporal
    int tile_store;          // the 16 rows of a tile are 16 * out_cols contiguous floats (ld_out == out_cols == 32,
                             // 16-byte aligned): they go through LDS and out as two 1 KB stores per wave
    unsigned swz_mask;       // row r of out lives at swizzled_row(r, swz_mask): 0 = vertex order (common.hpp)
    const uint32_t* rows;    // nullptr, or one bit per row of x: clear = the row counts as zeros and is not read
};

template <int VW, int MT, int CU, bool kRows>
__global__ __launch_bounds__(kUpdateThreads) void dense_rows_kernel(RowsArgs a)
{
    extern __shared__ __align__(16) float w_lds[];   // [MT][chunks_p][64 lanes][VW]
    const int chunks = (a.K + 4 * VW - 1) / (4 * VW);
    const int chunks_p = (chunks + CU - 1) / CU * CU;
    for (int idx = threadIdx.x; idx < MT * chunks_p * kWave * VW; idx += kUpdateThreads) {
        const int v = idx % VW;
        const int l = (idx / VW) % kWave;
        const int t = (idx / (VW * kWave)) % chunks_p;
        const int mt = idx / (VW * kWave * chunks_p);
        const int k = (4 * t + l / 16) * VW + v;
        const int m = mt * 16 + l % 16;
        w_lds[idx] = (k < a.K && m < a.M) ? a.w[k * a.sk + m * a.sm] : 0.f;
    }
    __syncthreads();

    const int lane = lane_id();
    const int wave = threadIdx.x / kWave;
    const int i = lane % 16, j = lane / 16;
    const long long tiles = (a.n + kTileRows - 1) / kTileRows;
    for (long long tile = static_cast<long long>(blockIdx.x) * kUpdateWaves + wave; tile < tiles;
         tile += static_cast<long long>(gridDim.x) * kUpdateWaves) {
        const long long r = tile * kTileRows + i;
        const bool row_ok = r < a.n;
        bool live = row_ok;
        if constexpr (kRows) live = row_ok && ((a.rows[r >> 5] >> (r & 31)) & 1u);
        const bool dead = row_ok && !live;               // a row the bitmap leaves out: counts as zeros
        // rows past the end read the last row and store nothing; a row the bitmap leaves out reads row 0 instead of its
        // own (every load stays unconditional) and its values are replaced by zeros
        const long long rc = live ? r : (row_ok ? 0 : a.n - 1);
        const float* __restrict__ xrow = a.x + rc * a.ld_x;
        floatx4 acc[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[mt] = floatx4{0.f, 0.f, 0.f, 0.f};

        for (int t0 = 0; t0 < chunks_p; t0 += CU) {
            float x[CU][VW];
#pragma unroll
            for (int u = 0; u < CU; ++u) load_row_piece<VW>(x[u], xrow, (4 * (t0 + u) + j) * VW, a.K, a.relu_in != 0);
            if constexpr (kRows) {
#pragma unroll
                for (int u = 0; u < CU; ++u)
#pragma unroll
                    for (int v = 0; v < VW; ++v) x[u][v] = dead ? 0.f : x[u][v];
            }
#pragma unroll
            for (int u = 0; u < CU; ++u) {
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    const float* wp = w_lds + ((mt * chunks_p + t0 + u) * kWave + lane) * VW;
                    float wv[VW];
                    if constexpr (VW == 4) {
                        const float4 t = *reinterpret_cast<const float4*>(wp);
                        wv[0] = t.x; wv[1] = t.y; wv[2] = t.z; wv[3] = t.w;
                    } else if constexpr (VW == 2) {
                        const float2 t = *reinterpret_cast<const float2*>(wp);
                        wv[0] = t.x; wv[1] = t.y;
                    } else {
                        wv[0] = wp[0];
                    }
#pragma unroll
                    for (int v = 0; v < VW; ++v) acc[mt] = mfma16(wv[v], x[u][v], acc[mt]);
                }
            }
        }

        if constexpr (MT == 2) {
            // Rows of 32 floats: a lane holds 4 columns of one row per 16-column tile, so a store instruction would
            // write one half of each of 16 lines.  The tile goes through the wave's LDS area instead and leaves as
            // 2 KB of consecutive 16-byte stores.  In the table's row order the 16 rows of a tile stay one aligned
            // block of 16 rows, permuted by the low bits of the XOR term (the same for all rows of the tile).
            if (a.tile_store) {
                __shared__ __align__(16) float o_lds[kUpdateWaves][16 * 32];
                float* __restrict__ ot = o_lds[wave];
                const long long r0 = tile * kTileRows;
                const unsigned x = (static_cast<unsigned>(r0) >> kRowSwizzleShift) & a.swz_mask;
                const float s = (row_ok && a.scale) ? a.scale[r] : 1.f;
                const int p = i ^ static_cast<int>(x & 15u);              // place of row r0 + i in the block
#pragma unroll
                for (int mt = 0; mt < 2; ++mt) {
                    const int m0 = mt * 16 + 4 * j;
                    float y[4] = {acc[mt][0] * s, acc[mt][1] * s, acc[mt][2] * s, acc[mt][3] * s};
                    if (a.relu_ref && live) {
                        const float* __restrict__ ref = a.relu_ref + r * a.ld_ref;
#pragma unroll
                        for (int v = 0; v < 4; ++v)
                            if (m0 + v < a.M && !(ref[m0 + v] > 0.f)) y[v] = 0.f;
                    }
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        if (m0 + v >= a.M) y[v] = 0.f;
                    *reinterpret_cast<float4*>(ot + p * 32 + m0) = make_float4(y[0], y[1], y[2], y[3]);
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                const long long b0 = static_cast<long long>((static_cast<unsigned>(r0) ^ (x & ~15u)));   // first row of the block
                float* __restrict__ obase = a.out + b0 * 32;
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int q = h * kWave + lane;                        // 16-byte vector of the 2 KB block
                    const int prow = q >> 3;                               // its row inside the block
                    if (r0 + (prow ^ static_cast<int>(x & 15u)) < a.n)
                        *reinterpret_cast<float4*>(obase + q * 4) = *reinterpret_cast<const float4*>(ot + q * 4);
                }
                __builtin_amdgcn_wave_barrier();                           // the area is rewritten by the next tile
                continue;
            }
        }
        if (!row_ok) continue;
        const float s = a.scale ? a.scale[r] : 1.f;
        float* __restrict__ orow = a.out + static_cast<long long>(swizzled_row(static_cast<unsigned>(r), a.swz_mask)) * a.ld_out;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m0 = mt * 16 + 4 * j;
            if (m0 >= a.out_cols) continue;
            float y[4] = {acc[mt][0] * s, acc[mt][1] * s, acc[mt][2] * s, acc[mt][3] * s};
            if (a.relu_ref && live) {
                const float* __restrict__ ref = a.relu_ref + r * a.ld_ref;
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (m0 + v < a.M && !(ref[m0 + v] > 0.f)) y[v] = 0.f;
            }
#pragma unroll
            for (int v = 0; v < 4; ++v)
                if (m0 + v >= a.M) y[v] = 0.f;        // padding columns hold exact zeros
            if (a.vec_store && m0 + 4 <= a.out_cols) {
                if (a.vec_store == 2) {      // wide result rows are written once and not read back soon
                    const floatx4 o = {y[0], y[1], y[2], y[3]};
                    __builtin_nontemporal_store(o, reinterpret_cast<floatx4*>(orow + m0));
                } else {
                    *reinterpret_cast<float4*>(orow + m0) = make_float4(y[0], y[1], y[2], y[3]);
                }
            } else {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (m0 + v < a.out_cols) orow[m0 + v] = y[v];
            }
        }
    }
}

template <int VW, int MT>
static hipError_t launch_rows_cu(const RowsArgs& a, int cu, unsigned blocks, size_t lds, hipStream_t stream)
{
#define EPPGCN_ROWS(CU_)                                                                                                \
    do {                                                                                                               \
        if (a.rows) hipLaunchKernelGGL((dense_rows_kernel<VW, MT, CU_, true>), dim3(blocks), dim3(kUpdateThreads), lds, stream, a); \
        else hipLaunchKernelGGL((dense_rows_kernel<VW, MT, CU_, false>), dim3(blocks), dim3(kUpdateThreads), lds, stream, a);       \
    } while (0)
    if (cu == 4) EPPGCN_ROWS(4);
    else if (cu == 2) EPPGCN_ROWS(2);
    else EPPGCN_ROWS(1);
#undef EPPGCN_ROWS
    return hipGetLastError();
}

template <int VW>
static hipError_t launch_rows_mt(const RowsArgs& a, int mt, int cu, unsigned blocks, size_t lds, hipStream_t stream)
{
    switch (mt) {
        case 1: return launch_rows_cu<VW, 1>(a, cu, blocks, lds, stream);
        case 2: return launch_rows_cu<VW, 2>(a, cu, blocks, lds, stream);
        case 4: return launch_rows_cu<VW, 4>(a, cu, blocks, lds, stream);
        default: return launch_rows_cu<VW, 8>(a, cu, blocks, lds, stream);
    }
}

// out[r, 0:out_cols] = scale[r] * (act(X[r, 0:K]) * Wop)[0:M] (zero beyond M), optionally masked by
// relu_ref.  Wop(k, m) = w[k*sk + m*sm].  Returns kErrInvalidArgument when K is too large for the
// operand to fit the LDS (the caller then has to use a general GEMM).
int launch_dense_rows(float* out, int ld_out, int out_cols, const float* x, int ld_x, const float* w, long long sk,
                      long long sm, const float* scale, const float* relu_ref, int ld_ref, int relu_in,
                      long long n, int K, int M, hipStream_t stream, unsigned swz_mask, const uint32_t* rows)
{
    if (n == 0 || out_cols == 0) return kOk;
    const uintptr_t xa = reinterpret_cast<uintptr_t>(x);
    const int vw = (ld_x % 4 == 0 && xa % 16 == 0) ? 4 : (ld_x % 2 == 0 && xa % 8 == 0) ? 2 : 1;
    const int chunks = (K + 4 * vw - 1) / (4 * vw);
    const int cu = chunks >= 3 ? 4 : chunks;
    const int chunks_p = (chunks + cu - 1) / cu * cu;
    const size_t lds_per_tile = static_cast<size_t>(chunks_p) * kWave * vw * sizeof(float);
    if (lds_per_tile > kMaxOperandLds) {
        set_error("dense update: inner dimension too large for the on-chip operand buffer");
        return kErrInvalidArgument;
    }
    int mt_cap = 8;                                     // 16-column tiles one launch covers
    while (mt_cap > 1 && lds_per_tile * mt_cap > kMaxOperandLds) mt_cap /= 2;
    const long long tiles = (n + kTileRows - 1) / kTileRows;
    long long blocks = (tiles + kUpdateWaves - 1) / kUpdateWaves;
    if (blocks > 256 * 8) blocks = 256 * 8;
    for (int c0 = 0; c0 < out_cols; c0 += 16 * mt_cap) {
        const int cols = out_cols - c0 < 16 * mt_cap ? out_cols - c0 : 16 * mt_cap;
        int mt = 1;
        while (16 * mt < cols) mt *= 2;
        RowsArgs a;
        a.out = out + c0;
        a.x = x;
        a.w = w + c0 * sm;
        a.scale = scale;
        a.relu_ref = relu_ref ? relu_ref + c0 : nullptr;
        a.n = n;
        a.sk = sk;
        a.sm = sm;
        a.ld_out = ld_out;
        a.out_cols = cols;
        a.ld_x = ld_x;
        a.ld_ref = ld_ref;
        a.K = K;
        a.M = M - c0 > 0 ? (M - c0 < cols ? M - c0 : cols) : 0;
        a.relu_in = relu_in;
        a.swz_mask = swz_mask;
        a.rows = rows;
        a.vec_store = (ld_out % 4 == 0 && reinterpret_cast<uintptr_t>(a.out) % 16 == 0) ? 1 : 0;
        // measured at 4.2 M rows: a [N, 96] result 0.63 -> 0.47 ms with non-temporal stores, [N, 16] and
        // [N, 32] results unchanged or slower
        if (a.vec_store && out_cols >= 64) a.vec_store = 2;
        a.tile_store = (a.vec_store && ld_out == 32 && cols == 32 && c0 == 0 && n < (1ll << 32)) ? 1 : 0;
        const size_t lds = lds_per_tile * mt;
        hipError_t e;
        if (vw == 4) e = launch_rows_mt<4>(a, mt, cu, static_cast<unsigned>(blocks), lds, stream);
        else if (vw == 2) e = launch_rows_mt<2>(a, mt, cu, static_cast<unsigned>(blocks), lds, stream);
        else e = launch_rows_mt<1>(a, mt, cu, static_cast<unsigned>(blocks), lds, stream);
        if (e != hipSuccess) return hip_fail(e, "dense rows kernel launch");
    }
    return kOk;
}

// ---------------------------------------------------------------- weight kernel
// partial[blockIdx.x][k][d] = sum over the block's rows of act(X[r, k]) * G[r, d]
template <int KTB, int DT>
__global__ __launch_bounds__(kUpdateThreads) void dense_weight_kernel(float* __restrict__ partial,
                                                                      const float* __restrict__ x, int ld_x,
                                                                      const float* __restrict__ g, int ld_g,
                                                                      int relu_in, long long n, int K, int D,
                                                                      long long rows_per_wave,
                                                                      const uint32_t* __restrict__ rows)
{
    __shared__ float red[kUpdateWaves][KTB * DT * 4 * kWave];
    const int lane = lane_id();
    const int wave = threadIdx.x / kWave;
    const int i = lane % 16, j = lane / 16;
    const int k0 = blockIdx.y * KTB * 16;
    floatx4 acc[KTB][DT];
#pragma unroll
    for (int kt = 0; kt < KTB; ++kt)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) acc[kt][dt] = floatx4{0.f, 0.f, 0.f, 0.f};

    const long long wave_id = static_cast<long long>(blockIdx.x) * kUpdateWaves + wave;
    const long long r_begin = wave_id * rows_per_wave;
    long long r_end = r_begin + rows_per_wave;
    if (r_end > n) r_end = n;
    for (long long r0 = r_begin; r0 < r_end; r0 += 16) {
        const unsigned bits = tile_row_bits(rows, r0);
        if (bits == 0u) continue;                       // wave-uniform: none of the 16 rows contributes
        float av[4][KTB], bv[4][DT];
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const long long row = r0 + 4 * s + j;
            const bool ok = row < r_end && ((bits >> (4 * s + j)) & 1u);
            const float* __restrict__ xr = x + (ok ? row : r_begin) * ld_x;
            const float* __restrict__ gr = g + (ok ? row : r_begin) * ld_g;
#pragma unroll
            for (int kt = 0; kt < KTB; ++kt) {
                const int k = k0 + kt * 16 + i;
                float t = (ok && k < K) ? xr[k] : 0.f;
                av[s][kt] = relu_in ? fmaxf(t, 0.f) : t;
            }
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const int d = dt * 16 + i;
                bv[s][dt] = (ok && d < D) ? gr[d] : 0.f;
            }
        }
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int kt = 0; kt < KTB; ++kt)
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) acc[kt][dt] = mfma16(av[s][kt], bv[s][dt], acc[kt][dt]);
    }

#pragma unroll
    for (int kt = 0; kt < KTB; ++kt)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int v = 0; v < 4; ++v) red[wave][((kt * DT + dt) * 4 + v) * kWave + lane] = acc[kt][dt][v];
    __syncthreads();
    float* __restrict__ mine = partial + static_cast<size_t>(blockIdx.x) * K * D;
    for (int e = threadIdx.x; e < KTB * DT * 4 * kWave; e += kUpdateThreads) {
        float sum = red[0][e];
#pragma unroll
        for (int w = 1; w < kUpdateWaves; ++w) sum += red[w][e];
        const int l = e % kWave;
        const int v = (e / kWave) % 4;
        const int dt = (e / (4 * kWave)) % DT;
        const int kt = e / (4 * kWave * DT);
        const int k = k0 + kt * 16 + 4 * (l / 16) + v;
        const int d = dt * 16 + l % 16;
        if (k < K && d < D) mine[static_cast<size_t>(k) * D + d] = sum;
    }
}

// dw[e] = sum over blocks of partial[b][e], added in a fixed order: 16 slices of a workgroup take every 16th block
// each (four running sums per slice), then the 16 slice sums are added as a tree
constexpr int kReduceSlices = 16;
__global__ __launch_bounds__(64 * kReduceSlices) void reduce_partials_kernel(float* __restrict__ dw,
                                                                             const float* __restrict__ partial,
                                                                             int num_blocks, int count)
{
    __shared__ float red[kReduceSlices][64];
    const int col = threadIdx.x % 64;
    const int e = blockIdx.x * 64 + col;
    const int slice = threadIdx.x / 64;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    if (e < count) {
        int b = slice;
        for (; b + 3 * kReduceSlices < num_blocks; b += 4 * kReduceSlices) {
            s0 += partial[static_cast<size_t>(b) * count + e];
            s1 += partial[static_cast<size_t>(b + kReduceSlices) * count + e];
            s2 += partial[static_cast<size_t>(b + 2 * kReduceSlices) * count + e];
            s3 += partial[static_cast<size_t>(b + 3 * kReduceSlices) * count + e];
        }
        for (; b < num_blocks; b += kReduceSlices) s0 += partial[static_cast<size_t>(b) * count + e];
    }
    red[slice][col] = (s0 + s1) + (s2 + s3);
    __syncthreads();
#pragma unroll
    for (int half = kReduceSlices / 2; half >= 1; half /= 2) {
        if (slice < half) red[slice][col] += red[slice + half][col];
        __syncthreads();
    }
    if (slice == 0 && e < count) dw[e] = red[0][col];
}

static int weight_blocks(long long n)
{
    long long b = (n + 63) / 64;                         // at least 16 rows per wave
    if (b > kMaxWeightBlocks) b = kMaxWeightBlocks;
    return static_cast<int>(b < 1 ? 1 : b);
}

size_t update_workspace_bytes(long long n, int K, int D)
{
    if (n <= 0 || K <= 0 || D <= 0) return 0;
    return static_cast<size_t>(weight_blocks(n)) * K * D * sizeof(float);
}

template <int KTB, int DT>
static hipError_t launch_weight(float* partial, const float* x, int ld_x, const float* g, int ld_g, int relu_in,
                                long long n, int K, int D, long long rows_per_wave, int blocks, hipStream_t stream,
                                const uint32_t* rows)
{
    const int ktiles = (K + 15) / 16;
    hipLaunchKernelGGL((dense_weight_kernel<KTB, DT>), dim3(blocks, (ktiles + KTB - 1) / KTB), dim3(kUpdateThreads), 0,
                       stream, partial, x, ld_x, g, ld_g, relu_in, n, K, D, rows_per_wave, rows);
    return hipGetLastError();
}

// dw[K, D] = act(X[N, K])^T * G[N, D]; D <= 64.
int launch_dense_weight(float* dw, const float* x, int ld_x, const float* g, int ld_g, int relu_in, long long n,
                        int K, int D, void* workspace, hipStream_t stream, const uint32_t* rows)
{
    if (K == 0 || D == 0) return kOk;
    if (n == 0) {
        return launch_zero_words(dw, static_cast<size_t>(K) * D, stream);
    }
    if (D > 64) {
        set_error("dense update: more than 64 gradient columns are not supported by the weight kernel");
        return kErrInvalidArgument;
    }
    const int blocks = weight_blocks(n);
    const long long waves = static_cast<long long>(blocks) * kUpdateWaves;
    const long long rows_per_wave = ((n + waves - 1) / waves + 15) / 16 * 16;
    float* partial = static_cast<float*>(workspace);
    const int dt = D <= 16 ? 1 : D <= 32 ? 2 : 4;
    const int ktiles = (K + 15) / 16;
    int ktb = 8 / dt;
    while (ktb > 1 && ktb / 2 >= ktiles) ktb /= 2;
    hipError_t e;
#define EPPGCN_W(KTB_, DT_) launch_weight<KTB_, DT_>(partial, x, ld_x, g, ld_g, relu_in, n, K, D, rows_per_wave, blocks, stream, rows)
    if (dt == 1) e = ktb == 8 ? EPPGCN_W(8, 1) : ktb == 4 ? EPPGCN_W(4, 1) : ktb == 2 ? EPPGCN_W(2, 1) : EPPGCN_W(1, 1);
    else if (dt == 2) e = ktb == 4 ? EPPGCN_W(4, 2) : ktb == 2 ? EPPGCN_W(2, 2) : EPPGCN_W(1, 2);
    else e = ktb == 2 ? EPPGCN_W(2, 4) : EPPGCN_W(1, 4);
#undef EPPGCN_W
    if (e != hipSuccess) return hip_fail(e, "dense weight kernel launch");
    const int count = K * D;
    hipLaunchKernelGGL(reduce_partials_kernel, dim3((count + 63) / 64), dim3(64 * kReduceSlices), 0, stream, dw, partial, blocks, count);
    EPPGCN_HIP(hipGetLastError());
    return kOk;
}

// ---------------------------------------------------------------- input and weight gradient in one pass
// dX[r, k] = [act'(X[r, k])] * sum_d G[r, d] * W[k, d]   and   dW[k, d] = sum_r act(X[r, k]) * G[r, d]
// for a narrow layer (K <= 16 inputs, D <= 32 gradient columns): both products read G and X, so a wave that owns a
// contiguous range of rows does both for every 16 rows it loads - G and X come from HBM once instead of twice.
// The 16 rows of G and of X are contiguous in memory (64 D and 64 K bytes): the wave copies them into its own LDS
// area with full 16-byte loads (three load instructions per step at K = 16, D = 22, where the operand layouts of
// the two products would take twenty narrow ones) and both products read their operands from there; the next
// step's rows are requested before the current step's products start.  Each product is accumulated exactly as
// dense_rows_kernel / dense_weight_kernel accumulate it (same tiles, same order of additions, same block sums), so
// the results equal those of the two separate launches bit for bit.
struct BackwardArgs {
    float* dx;               // [N, K]
    float* partial;          // [gridDim.x][K * D] block sums of dW
    const float* x;          // [N, K] layer input, 16-byte aligned
    const float* g;          // [N, D] gradient of the layer's product, 16-byte aligned
    const float* w;          // [K, D]
    long long n, rows_per_wave;
    int K, D;
    int relu_in;             // the layer applied max(x, 0) to its input
    int vec_store;           // rows of dx are 16-byte aligned
    const uint32_t* rows;    // nullptr, or one bit per row: clear = the row of g counts as zeros, it and its row of x are not read
};

constexpr int kBackMaxK = 16, kBackMaxD = 32;

template <int VW, int DT>
__global__ __launch_bounds__(kUpdateThreads) void dense_backward_kernel(BackwardArgs a)
{
    constexpr int CH = 4 * DT / VW;                          // steps of 4 * VW gradient columns that cover 16 * DT
    constexpr int kGVecs = 16 * 16 * DT / 4 / kWave;         // 16-byte vectors per lane that cover 16 rows of G
    __shared__ __align__(16) float w_lds[CH * kWave * VW];   // operand of the dX product, element (d, k) = w[k, d]
    __shared__ __align__(16) float g_lds[kUpdateWaves][16 * 16 * DT];
    __shared__ __align__(16) float x_lds[kUpdateWaves][16 * kBackMaxK];
    __shared__ float red[kUpdateWaves][DT * 4 * kWave];
    for (int idx = threadIdx.x; idx < CH * kWave * VW; idx += kUpdateThreads) {
        const int v = idx % VW;
        const int l = (idx / VW) % kWave;
        const int t = idx / (VW * kWave);
        const int d = (4 * t + l / 16) * VW + v;
        const int k = l % 16;
        w_lds[idx] = (d < a.D && k < a.K) ? a.w[k * a.D + d] : 0.f;
    }
    __syncthreads();

    const int lane = lane_id();
    const int wave = threadIdx.x / kWave;
    const int i = lane % 16, j = lane / 16;
    float* __restrict__ gt = g_lds[wave];
    float* __restrict__ xt = x_lds[wave];
    floatx4 accw[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) accw[dt] = floatx4{0.f, 0.f, 0.f, 0.f};

    const long long wave_id = static_cast<long long>(blockIdx.x) * kUpdateWaves + wave;
    const long long r_begin = wave_id * a.rows_per_wave;
    long long r_end = r_begin + a.rows_per_wave;
    if (r_end > a.n) r_end = a.n;

    // 16 rows from row r0 on (fewer at the end of the matrix; what lies past the wave's own range is loaded but
    // never used): G as kGVecs vectors per lane, X as one
    // which of the tile's 16 rows a lane's vectors touch (a 16-byte vector can lie across two rows): the same
    // for every tile, so worked out once.  A vector is fetched when one of its rows has its bit set.
    floatx4 gv[kGVecs], xv;
    unsigned gneed[kGVecs], xneed;
    auto rows_of = [](int off, int width) {
        const int ra = off / width, rb = (off + 3) / width;
        return (ra < 16 ? 1u << ra : 0u) | (rb < 16 ? 1u << rb : 0u);
    };
#pragma unroll
    for (int q = 0; q < kGVecs; ++q) gneed[q] = rows_of((q * kWave + lane) * 4, a.D);
    xneed = rows_of(lane * 4, a.K);
    auto request = [&](long long r0, unsigned bits) {
        const long long rows = a.n - r0 < 16 ? a.n - r0 : 16;
        const float* __restrict__ gsrc = a.g + r0 * a.D;
        const float* __restrict__ xsrc = a.x + r0 * a.K;
        const int gcount = static_cast<int>(rows) * a.D, xcount = static_cast<int>(rows) * a.K;
#pragma unroll
        for (int q = 0; q < kGVecs; ++q) {
            const int off = (q * kWave + lane) * 4;
            if (!(gneed[q] & bits)) gv[q] = floatx4{0.f, 0.f, 0.f, 0.f};
            else if (off + 4 <= gcount) gv[q] = *reinterpret_cast<const floatx4*>(gsrc + off);
            else
#pragma unroll
                for (int c = 0; c < 4; ++c) gv[q][c] = off + c < gcount ? gsrc[off + c] : 0.f;
        }
        const int off = lane * 4;
        if (!(xneed & bits)) xv = floatx4{0.f, 0.f, 0.f, 0.f};
        else if (off + 4 <= xcount) xv = *reinterpret_cast<const floatx4*>(xsrc + off);
        else
#pragma unroll
            for (int c = 0; c < 4; ++c) xv[c] = off + c < xcount ? xsrc[off + c] : 0.f;
    };
    unsigned bits = 0u, bits_next = 0u;
    if (r_begin < r_end) {
        bits = tile_row_bits(a.rows, r_begin);
        request(r_begin, bits);
    }

    for (long long r0 = r_begin; r0 < r_end; r0 += 16, bits = bits_next) {
        const long long r = r0 + i;
        const bool row_ok = r < r_end;
        const int m0 = 4 * j;
        if (bits == 0u) {            // wave-uniform: no row of the tile carries a gradient; its rows of dX are zeros
            if (r0 + 16 < r_end) {
                bits_next = tile_row_bits(a.rows, r0 + 16);
                request(r0 + 16, bits_next);
            }
            if (row_ok && m0 < a.K) {
                float* __restrict__ orow = a.dx + r * a.K;
                if (a.vec_store && m0 + 4 <= a.K) {
                    *reinterpret_cast<float4*>(orow + m0) = make_float4(0.f, 0.f, 0.f, 0.f);
                } else {
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        if (m0 + v < a.K) orow[m0 + v] = 0.f;
                }
            }
            continue;
        }
        // the wave's LDS area is its own: its LDS operations execute in order, so the stores below come after the
        // previous step's reads without a barrier
#pragma unroll
        for (int q = 0; q < kGVecs; ++q) *reinterpret_cast<floatx4*>(gt + (q * kWave + lane) * 4) = gv[q];
        *reinterpret_cast<floatx4*>(xt + lane * 4) = xv;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (r0 + 16 < r_end) {                               // under way during this step's products
            bits_next = tile_row_bits(a.rows, r0 + 16);
            request(r0 + 16, bits_next);
        }

        // ---- dX for rows r0 .. r0 + 15: lane (i, j) takes VW consecutive gradient columns of row r0 + i per step
        // (a row whose bit is clear may share a fetched vector with a neighbour: its values are not used)
        const bool row_live = (bits >> i) & 1u;
        floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < CH; ++t) {
            const float* wp = w_lds + (t * kWave + lane) * VW;
#pragma unroll
            for (int v = 0; v < VW; ++v) {
                const int d = (4 * t + j) * VW + v;
                acc = mfma16(wp[v], (d < a.D && row_live) ? gt[i * a.D + d] : 0.f, acc);
            }
        }
        if (row_ok && m0 < a.K) {
            float y[4] = {acc[0], acc[1], acc[2], acc[3]};
            if (a.relu_in) {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (m0 + v < a.K && !(xt[i * a.K + m0 + v] > 0.f)) y[v] = 0.f;
            }
            float* __restrict__ orow = a.dx + r * a.K;
            if (a.vec_store && m0 + 4 <= a.K) {
                *reinterpret_cast<float4*>(orow + m0) = make_float4(y[0], y[1], y[2], y[3]);
            } else {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (m0 + v < a.K) orow[m0 + v] = y[v];
            }
        }
        // ---- dW: lane (i, j) supplies column i of X and columns i, 16 + i of G for rows r0 + 4 s + j
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const int lr = 4 * s + j;
            const bool ok = r0 + lr < r_end && ((bits >> lr) & 1u);
            const float t = (ok && i < a.K) ? xt[lr * a.K + i] : 0.f;
            const float av = a.relu_in ? fmaxf(t, 0.f) : t;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const int d = dt * 16 + i;
                accw[dt] = mfma16(av, (ok && d < a.D) ? gt[lr * a.D + d] : 0.f, accw[dt]);
            }
        }
    }

#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int v = 0; v < 4; ++v) red[wave][(dt * 4 + v) * kWave + lane] = accw[dt][v];
    __syncthreads();
    float* __restrict__ mine = a.partial + static_cast<size_t>(blockIdx.x) * a.K * a.D;
    for (int e = threadIdx.x; e < DT * 4 * kWave; e += kUpdateThreads) {
        float sum = red[0][e];
#pragma unroll
        for (int w = 1; w < kUpdateWaves; ++w) sum += red[w][e];
        const int l = e % kWave;
        const int v = (e / kWave) % 4;
        const int dt = e / (4 * kWave);
        const int k = 4 * (l / 16) + v;
        const int d = dt * 16 + l % 16;
        if (k < a.K && d < a.D) mine[static_cast<size_t>(k) * a.D + d] = sum;
    }
}

// Shapes the one-pass kernel covers.
bool dense_backward_fused_covers(int K, int D, const float* x, const float* g)
{
    return K >= 1 && K <= kBackMaxK && D >= 1 && D <= kBackMaxD &&
           (reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(g)) % 16 == 0;
}

// dx[N, K] and dw[K, D] of a layer out = act(X) * W from the gradient G[N, D] of the product, in one pass over X
// and G (dense_backward_fused_covers(K, D) holds; `workspace` as for launch_dense_weight).
int launch_dense_backward(float* dx, float* dw, const float* x, const float* g, const float* w, int relu_in,
                          long long n, int K, int D, void* workspace, hipStream_t stream, const uint32_t* rows)
{
    if (n == 0) return launch_zero_words(dw, static_cast<size_t>(K) * D, stream);
    const int blocks = weight_blocks(n);
    const long long waves = static_cast<long long>(blocks) * kUpdateWaves;
    BackwardArgs a;
    a.dx = dx;
    a.partial = static_cast<float*>(workspace);
    a.x = x;
    a.g = g;
    a.w = w;
    a.n = n;
    a.rows_per_wave = ((n + waves - 1) / waves + 15) / 16 * 16;
    a.K = K;
    a.D = D;
    a.relu_in = relu_in;
    a.vec_store = (K % 4 == 0 && reinterpret_cast<uintptr_t>(dx) % 16 == 0) ? 1 : 0;
    a.rows = rows;
    const int vw = D % 4 == 0 ? 4 : D % 2 == 0 ? 2 : 1;        // the order of additions of dense_rows_kernel for aligned g
    const int dt = D <= 16 ? 1 : 2;
#define EPPGCN_B(VW_, DT_) hipLaunchKernelGGL((dense_backward_kernel<VW_, DT_>), dim3(blocks), dim3(kUpdateThreads), 0, stream, a)
    if (vw == 4) { if (dt == 1) EPPGCN_B(4, 1); else EPPGCN_B(4, 2); }
    else if (vw == 2) { if (dt == 1) EPPGCN_B(2, 1); else EPPGCN_B(2, 2); }
    else { if (dt == 1) EPPGCN_B(1, 1); else EPPGCN_B(1, 2); }
#undef EPPGCN_B
    EPPGCN_HIP(hipGetLastError());
    const int count = K * D;
    hipLaunchKernelGGL(reduce_partials_kernel, dim3((count + 63) / 64), dim3(64 * kReduceSlices), 0, stream, dw, a.partial, blocks, count);
    EPPGCN_HIP(hipGetLastError());
    return kOk;
}

}  // namespace eppgcn
