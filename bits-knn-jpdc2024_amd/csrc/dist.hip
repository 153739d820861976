// Distance matrices for gfx950.
//
//  BITSKNN_DIST_L2          sum_t (q_t - p_t)^2 with one fused multiply-add per dimension, in
//                           dimension order: the arithmetic of the reference's default distance
//                           (include/bits/distance/abstract_gemm.cuh:59-100), reproducible bit for
//                           bit.  No matrix cores: the subtraction sits inside the contraction.
//  BITSKNN_DIST_PARTIAL_L2  ||p||^2 - 2 q.p (abstract_gemm.cuh:108-170) and
//  BITSKNN_DIST_EXPANDED    -2 q.p, then + ||p||^2 (src/distance/cublas_distance.cu:111-186):
//                           the q.p contraction runs on fp32 MFMA (v_mfma_f32_32x32x2_f32), the
//                           point norms are accumulated in dimension order next to it, and the
//                           epilogue writes fl(norm - 2*dot) once.  Both names give the same
//                           value here.
//
// Inputs are dim-major (component t of vector v at base[t*stride + v]), the output is the
// row-major q x n matrix; all index arithmetic on the output is 64-bit (q*n reaches 2^32).

#include <type_traits>

#include <initializer_list>

#include "common.hpp"
#include "dist_split.hpp"

namespace bitsknn
{
namespace
{

typedef float vfloat4 __attribute__((ext_vector_type(4)));
typedef float vfloat16 __attribute__((ext_vector_type(16)));

// ---------------------------------------------------------------------------------------------
// exact L2: every wave owns QW queries (wave-uniform operands), every lane 4 consecutive points
// ---------------------------------------------------------------------------------------------
constexpr int L2_QW = 8;                  // queries per wave
constexpr int L2_WAVES = 4;               // waves per workgroup
constexpr int L2_PT = WAVE * 4;           // points per workgroup
constexpr int L2_QT = L2_QW * L2_WAVES;   // queries per workgroup

template <bool ALIGNED>
__global__ void __launch_bounds__(WAVE* L2_WAVES)
    dist_l2_kernel(int dim, size_t q, size_t n, const float* __restrict__ queries, size_t qs,
                   const float* __restrict__ points, size_t ps, float* __restrict__ dist, size_t ds)
{
    const int lane = static_cast<int>(threadIdx.x) & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) / WAVE);
    const size_t j0 = static_cast<size_t>(blockIdx.x) * L2_PT + static_cast<size_t>(lane) * 4;
    const size_t i0 = static_cast<size_t>(blockIdx.y) * L2_QT + static_cast<size_t>(wave) * L2_QW;
    if (i0 >= q)
    {
        return;
    }

    float acc[L2_QW][4];
#pragma unroll
    for (int a = 0; a < L2_QW; ++a)
    {
#pragma unroll
        for (int b = 0; b < 4; ++b)
        {
            acc[a][b] = 0.0F;
        }
    }

    // queries beyond the end are clamped for loading and skipped when storing
    size_t qi[L2_QW];
#pragma unroll
    for (int a = 0; a < L2_QW; ++a)
    {
        qi[a] = i0 + a < q ? i0 + a : q - 1;
    }

    for (int t = 0; t < dim; ++t)
    {
        const float* __restrict__ prow = points + static_cast<size_t>(t) * ps;
        float p[4];
        if (ALIGNED && j0 + 4 <= n)
        {
            const vfloat4 x = *reinterpret_cast<const vfloat4*>(prow + j0);
            p[0] = x.x;
            p[1] = x.y;
            p[2] = x.z;
            p[3] = x.w;
        }
        else
        {
#pragma unroll
            for (int b = 0; b < 4; ++b)
            {
                p[b] = j0 + b < n ? prow[j0 + b] : 0.0F;
            }
        }
        const float* __restrict__ qrow = queries + static_cast<size_t>(t) * qs;
#pragma unroll
        for (int a = 0; a < L2_QW; ++a)
        {
            const float qv = qrow[qi[a]];
#pragma unroll
            for (int b = 0; b < 4; ++b)
            {
                const float diff = qv - p[b];
                acc[a][b] = __builtin_fmaf(diff, diff, acc[a][b]);
            }
        }
    }

#pragma unroll
    for (int a = 0; a < L2_QW; ++a)
    {
        if (i0 + a < q)
        {
            float* __restrict__ out = dist + (i0 + a) * ds + j0;
            if (ALIGNED && j0 + 4 <= n)
            {
                vfloat4 x;
                x.x = acc[a][0];
                x.y = acc[a][1];
                x.z = acc[a][2];
                x.w = acc[a][3];
                __builtin_nontemporal_store(x, reinterpret_cast<vfloat4*>(out));
            }
            else
            {
#pragma unroll
                for (int b = 0; b < 4; ++b)
                {
                    if (j0 + b < n)
                    {
                        out[b] = acc[a][b];
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// ||p||^2 - 2 q.p on fp32 MFMA.
//
// Workgroup tile 128 queries x 128 points, 4 waves as 2 x 2, each wave 64 x 64 = 2 x 2 MFMA
// tiles of 32 x 32.  The dimensions are walked in slabs of KT; a slab of both operands is staged
// in LDS exactly as it lies in memory (dim-major rows of 128 consecutive vectors), which is
// already the operand layout of v_mfma_f32_32x32x2_f32: lane l supplies row/column l%32 of
// dimension t0 + l/32.
// ---------------------------------------------------------------------------------------------
constexpr int MM_TILE = 128;
constexpr int MM_KT = 16;

__global__ void __launch_bounds__(256)
    dist_mfma_kernel(int dim, size_t q, size_t n, const float* __restrict__ queries, size_t qs,
                     const float* __restrict__ points, size_t ps, float* __restrict__ dist, size_t ds)
{
    __shared__ float q_lds[2][MM_KT][MM_TILE];
    __shared__ float p_lds[2][MM_KT][MM_TILE];
    __shared__ float norm_lds[MM_TILE];

    const int t = static_cast<int>(threadIdx.x);
    const int lane = t & (WAVE - 1);
    const int wave = t / WAVE;
    const int wm = wave / 2; // wave row: queries wm*64 .. +63 of the tile
    const int wn = wave % 2; // wave column: points wn*64 .. +63 of the tile
    // query tiles vary fastest over the grid so that workgroups sharing a point tile run together
    const size_t i_tile = static_cast<size_t>(blockIdx.x) * MM_TILE;
    const size_t j_tile = static_cast<size_t>(blockIdx.y) * MM_TILE;

    vfloat16 acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; ++a)
    {
#pragma unroll
        for (int b = 0; b < 2; ++b)
        {
#pragma unroll
            for (int r = 0; r < 16; ++r)
            {
                acc[a][b][r] = 0.0F;
            }
        }
    }

    // staging: thread t copies column (t % 128) of rows (t / 128) + 2*s, s = 0..KT/2-1
    const int col = t % MM_TILE;
    const int row0 = t / MM_TILE;
    const bool q_ok = i_tile + col < q;
    const bool p_ok = j_tile + col < n;
    float norm = 0.0F; // ||p||^2 of point `col`, accumulated in dimension order by threads t < 128

    // a slab travels global -> registers (before the MFMAs of the previous slab) -> LDS (after)
    float q_reg[MM_KT / 2];
    float p_reg[MM_KT / 2];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int s = 0; s < MM_KT / 2; ++s)
        {
            const int tt = k0 + row0 + 2 * s;
            q_reg[s] = 0.0F;
            p_reg[s] = 0.0F;
            if (tt < dim)
            {
                if (q_ok)
                {
                    q_reg[s] = queries[static_cast<size_t>(tt) * qs + i_tile + col];
                }
                if (p_ok)
                {
                    p_reg[s] = points[static_cast<size_t>(tt) * ps + j_tile + col];
                }
            }
        }
    };
    auto deposit = [&](int buf) {
#pragma unroll
        for (int s = 0; s < MM_KT / 2; ++s)
        {
            q_lds[buf][row0 + 2 * s][col] = q_reg[s];
            p_lds[buf][row0 + 2 * s][col] = p_reg[s];
        }
    };

    const int slabs = (dim + MM_KT - 1) / MM_KT;
    fetch(0);
    deposit(0);
    __syncthreads();
    for (int s = 0; s < slabs; ++s)
    {
        const int buf = s & 1;
        if (s + 1 < slabs)
        {
            fetch((s + 1) * MM_KT);
        }
        if (t < MM_TILE)
        {
#pragma unroll
            for (int r = 0; r < MM_KT; ++r)
            {
                const float pv = p_lds[buf][r][t];
                norm = __builtin_fmaf(pv, pv, norm);
            }
        }
#pragma unroll
        for (int kk = 0; kk < MM_KT; kk += 2)
        {
            const int r = kk + lane / 32;
            float av[2];
            float bv[2];
#pragma unroll
            for (int a = 0; a < 2; ++a)
            {
                av[a] = q_lds[buf][r][wm * 64 + a * 32 + (lane & 31)];
                bv[a] = p_lds[buf][r][wn * 64 + a * 32 + (lane & 31)];
            }
#pragma unroll
            for (int a = 0; a < 2; ++a)
            {
#pragma unroll
                for (int b = 0; b < 2; ++b)
                {
                    acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[a], bv[b], acc[a][b], 0, 0, 0);
                }
            }
        }
        if (s + 1 < slabs)
        {
            deposit(buf ^ 1);
        }
        __syncthreads();
    }
    if (t < MM_TILE)
    {
        norm_lds[t] = norm;
    }
    __syncthreads();

    // epilogue: element r of lane l is row 8*(r/4) + 4*(l/32) + r%4, column l%32 of the 32x32 tile
#pragma unroll
    for (int b = 0; b < 2; ++b)
    {
        const int jc = wn * 64 + b * 32 + (lane & 31);
        const size_t j = j_tile + jc;
        const float pn = norm_lds[jc];
#pragma unroll
        for (int a = 0; a < 2; ++a)
        {
#pragma unroll
            for (int r = 0; r < 16; ++r)
            {
                const size_t i = i_tile + wm * 64 + a * 32 + 8 * (r / 4) + 4 * (lane / 32) + (r % 4);
                if (i < q && j < n)
                {
                    __builtin_nontemporal_store(__builtin_fmaf(-2.0F, acc[a][b][r], pn),
                                                dist + i * ds + j);
                }
            }
        }
    }
}


// ---------------------------------------------------------------------------------------------
// ||p||^2 - 2 q.p on fp32 MFMA, query-resident form (dimensions up to 256).
//
// A workgroup of 4 waves owns QPW x 4 x 32 queries, whose fragments (q_0..q_{d-1}, 1, 1) stay in
// registers as the MFMA A operand, and walks over a range of points in stages of PT.  A stage is
// written to LDS once as the B operand: rows -2*p, then one row per staging thread of a point
// with its share of ||p||^2, so the product IS the distance and the epilogue is a plain store.
// In the 32 x 32 result a lane holds one point (column) and 16 queries (rows): for every register
// the two half-waves write two full 128-byte segments of the row-major output.
// ---------------------------------------------------------------------------------------------
template <int DP>
struct resident_geometry
{
    static constexpr int PT = DP <= 64 ? 128 : (DP <= 128 ? 64 : 32);
    static constexpr int TPP = 256 / PT;                  // staging threads per point
    static constexpr int NORM_ROWS = TPP > 2 ? TPP : 2;
    static constexpr int ROWS = DP + NORM_ROWS;
    static constexpr int STEPS = ROWS / 2;
    static constexpr int VPT = DP / TPP;                  // staged values per thread
    static constexpr int NT = PT / 32;                    // column tiles per stage
    static constexpr int QPW = DP <= 64 ? 2 : 1;          // 32-query row tiles per wave
    static constexpr int QB = 4 * 32 * QPW;               // queries per workgroup
    static constexpr int RANGE = 4096;                    // points per workgroup
};

// Covers queries q_first.. and points n_first.. of the matrix (the pipelined kernel below takes
// the interior, this one the ragged edges, or everything when the pipelined one does not apply).
// STREAMING: rows start on 128-byte boundaries (see the stores).
template <int DP, bool STREAMING>
__global__ void __launch_bounds__(256)
    dist_resident_kernel(int dim, size_t q, size_t n, const float* __restrict__ queries, size_t qs,
                         const float* __restrict__ points, size_t ps, float* __restrict__ dist, size_t ds,
                         size_t q_first, size_t n_first)
{
    using G = resident_geometry<DP>;
    constexpr int PT = G::PT;
    constexpr int TPP = G::TPP;
    constexpr int STEPS = G::STEPS;
    constexpr int VPT = G::VPT;
    constexpr int QPW = G::QPW;
    constexpr int STAGE_FLOATS = G::ROWS * PT;

    __shared__ float stages[2 * STAGE_FLOATS];

    const int t = static_cast<int>(threadIdx.x);
    const int lane = t & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(t / WAVE);
    const int half = lane / 32;
    const int col = lane & 31;
    const size_t wave_q0 =
        q_first + static_cast<size_t>(blockIdx.x) * G::QB + static_cast<size_t>(wave) * 32 * QPW;
    const size_t j_begin = n_first + static_cast<size_t>(blockIdx.y) * G::RANGE;
    const size_t j_end = j_begin + G::RANGE < n ? j_begin + G::RANGE : n;

    // query fragments: step s of this lane is row 2s + half; the norm rows are multiplied by 1
    float qf[QPW][STEPS];
#pragma unroll
    for (int a = 0; a < QPW; ++a)
    {
        const size_t i = wave_q0 + a * 32 + col;
#pragma unroll
        for (int s = 0; s < STEPS; ++s)
        {
            const int dd = 2 * s + half;
            float val = dd >= DP ? 1.0F : 0.0F;
            if (dd < dim && i < q)
            {
                val = queries[static_cast<size_t>(dd) * qs + i];
            }
            qf[a][s] = val;
        }
    }

    for (int i = t; i < 2 * STAGE_FLOATS; i += 256)
    {
        stages[i] = 0.0F;
    }
    __syncthreads();

    const int sp = t % PT;
    const int sd0 = t / PT;
    const bool whole_dim = dim == DP;
    float pre[VPT];
    auto fetch = [&](size_t base) {
        if (whole_dim && base + PT <= j_end)
        {
            const float* __restrict__ src = points + static_cast<size_t>(sd0) * ps + base + sp;
#pragma unroll
            for (int i = 0; i < VPT; ++i)
            {
                pre[i] = src[static_cast<size_t>(TPP * i) * ps];
            }
        }
        else
        {
            const size_t j = base + sp;
#pragma unroll
            for (int i = 0; i < VPT; ++i)
            {
                const int dd = sd0 + TPP * i;
                pre[i] = 0.0F;
                if (dd < dim && j < j_end)
                {
                    pre[i] = points[static_cast<size_t>(dd) * ps + j];
                }
            }
        }
    };
    auto deposit = [&](float* stage) {
        float share = 0.0F;
#pragma unroll
        for (int i = 0; i < VPT; ++i)
        {
            const int dd = sd0 + TPP * i;
            share = __builtin_fmaf(pre[i], pre[i], share);
            if (whole_dim || dd < dim)
            {
                stage[dd * PT + sp] = -2.0F * pre[i];
            }
        }
        stage[(DP + sd0) * PT + sp] = share;
    };

    auto multiply = [&](const float* stage, size_t base) {
#pragma unroll 1
        for (int nt = 0; nt < G::NT; ++nt)
        {
            vfloat16 acc[QPW];
#pragma unroll
            for (int a = 0; a < QPW; ++a)
            {
#pragma unroll
                for (int r = 0; r < 16; ++r)
                {
                    acc[a][r] = 0.0F;
                }
            }
            const float* brow = stage + half * PT + nt * 32 + col;
            // operands are requested from LDS one chunk of steps ahead of the multiplies that use them
            constexpr int CH = STEPS <= 17 ? STEPS : 8;
            float bv[2][CH];
#pragma unroll
            for (int s = 0; s < CH; ++s)
            {
                bv[0][s] = brow[2 * s * PT];
            }
#pragma unroll
            for (int c = 0; c < STEPS; c += CH)
            {
#pragma unroll
                for (int s = 0; s < CH; ++s)
                {
                    if (c + CH + s < STEPS)
                    {
                        bv[(c / CH + 1) & 1][s] = brow[2 * (c + CH + s) * PT];
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int s = 0; s < CH; ++s)
                {
                    if (c + s < STEPS)
                    {
#pragma unroll
                        for (int a = 0; a < QPW; ++a)
                        {
                            acc[a] = __builtin_amdgcn_mfma_f32_32x32x2f32(qf[a][c + s], bv[(c / CH) & 1][s],
                                                                          acc[a], 0, 0, 0);
                        }
                    }
                }
            }
            const size_t j = base + nt * 32 + col;
            if (j < j_end)
            {
#pragma unroll
                for (int a = 0; a < QPW; ++a)
                {
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                    {
                        const size_t i = wave_q0 + a * 32 + 8 * (r / 4) + 4 * half + (r % 4);
                        if (i < q)
                        {
                            // Rows that are not 128-byte aligned share cache lines between
                            // neighbouring tiles: ordinary stores let L2 merge the pieces, where
                            // streaming stores would write partial lines to memory.
                            if constexpr (STREAMING)
                            {
                                __builtin_nontemporal_store(acc[a][r], dist + i * ds + j);
                            }
                            else
                            {
                                dist[i * ds + j] = acc[a][r];
                            }
                        }
                    }
                }
            }
        }
    };

    if (j_begin >= j_end)
    {
        return;
    }
    fetch(j_begin);
    __builtin_amdgcn_s_waitcnt(0x0F70);
    deposit(stages);
    if (j_begin + PT < j_end)
    {
        fetch(j_begin + PT);
    }
    __syncthreads();
    int parity = 0;
    for (size_t base = j_begin; base < j_end; base += PT)
    {
        multiply(stages + parity * STAGE_FLOATS, base);
        parity ^= 1;
        if (base + PT < j_end)
        {
            deposit(stages + parity * STAGE_FLOATS);
            if (base + 2 * PT < j_end)
            {
                fetch(base + 2 * PT);
            }
        }
        __syncthreads();
    }
}

// f(integral_constant<int, BEGIN>) ... f(integral_constant<int, END - 1>), expanded by the front
// end so that register arrays are indexed by constants whatever the size of the body
template <int BEGIN, int END, typename F>
__device__ __forceinline__ void static_for(F&& f)
{
    if constexpr (BEGIN < END)
    {
        f(std::integral_constant<int, BEGIN>{});
        static_for<BEGIN + 1, END>(f);
    }
}

// ---------------------------------------------------------------------------------------------
// Pipelined form of the query-resident kernel for the interior of the matrix: whole blocks of
// 128 queries, whole stages of PT points, dimensions up to 128.
//
// On gfx950 a wave that issues matrix instructions back to back leaves no issue slots to the
// other waves of its SIMD, and vector-ALU instructions of the same wave are not overlapped with
// its matrix instructions; LDS and memory instructions are.  So the loop over stages keeps the
// vector ALU out of the way: one wave per SIMD, and between two multiplies only LDS reads and
// writes, buffer loads and buffer stores whose addresses are a constant lane offset plus a
// scalar offset.
//  * The -2 of -2 q.p is folded into the query fragment (the B operand, in registers); a stage in
//    LDS holds the raw point values and the staging threads' shares of ||p||^2 (A operand).
//  * With the points as A operand a lane holds, in four consecutive result registers, four
//    consecutive points of ONE query.  A finished stage (32 queries x PT points per wave) is
//    written to a per-wave LDS tile with 16-byte writes, read back row by row during the next
//    stage, and stored with 16-byte buffer stores: 512 contiguous bytes per row and half-wave.
//  * Point values of the next stage are requested with buffer loads during the first third of a
//    stage and written to LDS during the last third; the only vector instructions per stage are
//    the VPT multiply-adds of the norm shares, issued in one burst.
// Results are bit-identical to the plain kernel: same products (scaling by -2 is exact) added in
// the same order.
// ---------------------------------------------------------------------------------------------
template <int DP>
struct pipelined_geometry
{
    static constexpr int PT = DP <= 64 ? 128 : 64;       // points per stage
    static constexpr int TPP = 256 / PT;                  // staging threads per point
    static constexpr int ROWS = DP + TPP;                 // dimensions + norm shares
    static constexpr int STEPS = ROWS / 2;
    static constexpr int VPT = DP / TPP;                  // staged values per thread
    static constexpr int NT = PT / 32;                    // 32-point tiles per stage
    static constexpr int QB = 128;                        // queries per workgroup (32 per wave)
    static constexpr int TP = PT + 4;                     // row pitch of the result tile in LDS
    static constexpr int STAGE_FLOATS = ROWS * PT;
    static constexpr int LDS_FLOATS = 2 * STAGE_FLOATS + 4 * 32 * TP;
};

typedef unsigned int vuint4 __attribute__((ext_vector_type(4)));

template <int DP>
__global__ void __launch_bounds__(256)
    dist_pipelined_kernel(int dim, size_t q_full, size_t n_full, const float* __restrict__ queries, size_t qs,
                          const float* __restrict__ points, size_t ps, float* __restrict__ dist, size_t ds,
                          unsigned range)
{
    using G = pipelined_geometry<DP>;
    constexpr int PT = G::PT;
    constexpr int TPP = G::TPP;
    constexpr int STEPS = G::STEPS;
    constexpr int VPT = G::VPT;
    constexpr int NT = G::NT;
    constexpr int TP = G::TP;
    constexpr int SLOTS = STEPS * NT;   // one slot per multiply
    static_assert(SLOTS >= 16 && VPT <= SLOTS / 3);

    __shared__ float lds[G::LDS_FLOATS];
    float* const stages = lds;

    const int t = static_cast<int>(threadIdx.x);
    const int lane = t & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(t / WAVE);
    const int half = lane / 32;
    const int col = lane & 31;
    const size_t wave_q0 = static_cast<size_t>(blockIdx.x) * G::QB + static_cast<size_t>(wave) * 32;
    // `range` points (a multiple of PT) per workgroup
    const size_t j_begin = static_cast<size_t>(blockIdx.y) * range;
    const size_t j_end = j_begin + range < n_full ? j_begin + range : n_full;
    const int stage_count = static_cast<int>((j_end - j_begin) / PT);
    float* const tile = lds + 2 * G::STAGE_FLOATS + wave * 32 * TP;

    // B operand: step s of this lane is dimension 2s + half of query `col`, times -2; the norm
    // rows are multiplied by 1
    float qf[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; ++s)
    {
        const int dd = 2 * s + half;
        float val = dd >= DP ? 1.0F : 0.0F;
        if (dd < dim)
        {
            val = -2.0F * queries[static_cast<size_t>(dd) * qs + wave_q0 + col];
        }
        qf[s] = val;
    }

    // Buffer resources: base + constant lane offset + scalar offset.
    const auto point_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(points + j_begin), 0,
        static_cast<int>((static_cast<size_t>(dim) * ps - j_begin) * sizeof(float)), 0x00020000);
    const auto dist_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        dist + wave_q0 * ds + j_begin, 0, static_cast<int>((31 * ds + (j_end - j_begin)) * sizeof(float)),
        0x00020000);
    const int sp = t % PT;
    const int sd0 = t / PT;
    // a row of a finished stage is PT/4 16-byte pieces: one store instruction covers RPI rows
    constexpr int QPR = PT / 4;
    constexpr int RPI = WAVE / QPR;
    constexpr int NE = 32 / RPI;   // store instructions per stage
    const int store_lane_off =
        static_cast<int>((static_cast<size_t>(lane / QPR) * ds + 4 * (lane % QPR)) * sizeof(float));

    // Byte offset of value i of this thread (dimension sd0 + TPP*i of point sp) inside the point
    // resource; the stage is selected by the scalar offset.  The hardware checks only the lane
    // offset against the size of the resource, so dimensions dim .. DP-1 get an offset beyond it
    // and read as zero.
    int load_off[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i)
    {
        const int dd = sd0 + TPP * i;
        load_off[i] = dd < dim ? static_cast<int>((static_cast<size_t>(dd) * ps + sp) * sizeof(float)) : 0x7FFFFFF0;
    }
    float pre[VPT];
    auto request = [&](auto i_tag, int first) {
        constexpr int i = decltype(i_tag)::value;
        pre[i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                               point_rsrc, load_off[i], first * static_cast<int>(sizeof(float)), 0));
    };
    auto write_value = [&](auto i_tag, float* stage) {
        constexpr int i = decltype(i_tag)::value;
        stage[(sd0 + TPP * i) * PT + sp] = pre[i];
    };
    auto write_share = [&](float* stage) {
        float share = 0.0F;
#pragma unroll
        for (int i = 0; i < VPT; ++i)
        {
            share = __builtin_fmaf(pre[i], pre[i], share);
        }
        stage[(DP + sd0) * PT + sp] = share;
    };
    // row group e (rows RPI*e .. RPI*e + RPI-1 of the wave's 32 queries) of the finished stage at `first`
    auto read_rows = [&](auto e_tag) -> vfloat4 {
        constexpr int e = decltype(e_tag)::value;
        return *reinterpret_cast<const vfloat4*>(tile + (RPI * e + lane / QPR) * TP + 4 * (lane % QPR));
    };
    auto store_rows = [&](auto e_tag, vfloat4 rows, int first) {
        constexpr int e = decltype(e_tag)::value;
        const int scalar_off =
            static_cast<int>((static_cast<size_t>(RPI * e) * ds + static_cast<size_t>(first)) * sizeof(float));
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(vuint4, rows), dist_rsrc, store_lane_off,
                                               scalar_off, 2 /* non-temporal */);
    };

    vfloat16 acc[NT];
    // lane (query col, half) holds in acc[k][4g .. 4g+3] the points 32k + 8g + 4*half + 0..3
    auto park_results = [&]() {
        static_for<0, NT>([&](auto k_tag) {
            constexpr int k = decltype(k_tag)::value;
            static_for<0, 4>([&](auto g_tag) {
                constexpr int g = decltype(g_tag)::value;
                vfloat4 v;
                v[0] = acc[k][4 * g + 0];
                v[1] = acc[k][4 * g + 1];
                v[2] = acc[k][4 * g + 2];
                v[3] = acc[k][4 * g + 3];
                *reinterpret_cast<vfloat4*>(tile + col * TP + 32 * k + 8 * g + 4 * half) = v;
            });
        });
    };

    // One stage.  HAVE_PREV: the LDS tile holds the results of the stage before (at first - PT),
    // to be stored.  HAVE_NEXT: the stage after this one exists; its values are requested during
    // the first third of the multiplies and written to `stage_next` during the last third (the
    // middle third covers the latency of the loads).  Both are types: a branch between two
    // multiplies would cost an instruction fetch that nothing hides.
    auto run_stage = [&](auto prev_tag, auto next_tag, const float* stage, float* stage_next, int first) {
        constexpr bool have_prev = decltype(prev_tag)::value;
        constexpr bool have_next = decltype(next_tag)::value;
        constexpr int THIRD = SLOTS / 3;
        constexpr int STRIDE = SLOTS / NE;
        const float* arow = stage + half * PT + col;
        float av[2][NT];
        static_for<0, NT>([&](auto k_tag) { av[0][decltype(k_tag)::value] = arow[32 * decltype(k_tag)::value]; });
        vfloat4 rows;
        static_for<0, STEPS>([&](auto s_tag) {
            constexpr int s = decltype(s_tag)::value;
            static_for<0, NT>([&](auto k_tag) {
                constexpr int k = decltype(k_tag)::value;
                constexpr int slot = s * NT + k;
                if constexpr (s + 1 < STEPS)
                {
                    av[(s + 1) & 1][k] = arow[2 * (s + 1) * PT + 32 * k];
                }
                if constexpr (s == 0)
                {
                    vfloat16 zero;
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                    {
                        zero[r] = 0.0F;
                    }
                    acc[k] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[0][k], qf[0], zero, 0, 0, 0);
                }
                else
                {
                    acc[k] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[s & 1][k], qf[s], acc[k], 0, 0, 0);
                }
                if constexpr (have_prev && slot / STRIDE < NE)
                {
                    // row group slot / STRIDE of the previous stage: read here, stored half a stride on
                    if constexpr (slot % STRIDE == 0)
                    {
                        rows = read_rows(std::integral_constant<int, slot / STRIDE>{});
                    }
                    if constexpr (slot % STRIDE == STRIDE / 2)
                    {
                        store_rows(std::integral_constant<int, slot / STRIDE>{}, rows, first - PT);
                    }
                }
                if constexpr (have_next)
                {
                    if constexpr (slot < THIRD)
                    {
                        static_for<slot * VPT / THIRD, (slot + 1) * VPT / THIRD>(
                            [&](auto i_tag) { request(i_tag, first + PT); });
                    }
                    else if constexpr (slot >= SLOTS - THIRD)
                    {
                        constexpr int w = slot - (SLOTS - THIRD);
                        if constexpr (w == 0)
                        {
                            write_share(stage_next);
                        }
                        static_for<w * VPT / THIRD, (w + 1) * VPT / THIRD>(
                            [&](auto i_tag) { write_value(i_tag, stage_next); });
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            });
        });
        park_results();
    };

    if (stage_count <= 0)
    {
        return;
    }
    // prologue: stage 0 into LDS
    static_for<0, VPT>([&](auto i_tag) { request(i_tag, 0); });
    write_share(stages);
    static_for<0, VPT>([&](auto i_tag) { write_value(i_tag, stages); });
    lds_barrier();

    constexpr std::true_type yes{};
    constexpr std::false_type no{};
    for (int st = 0; st < stage_count; ++st)
    {
        const float* const stage = stages + (st & 1) * G::STAGE_FLOATS;
        float* const stage_next = stages + ((st & 1) ^ 1) * G::STAGE_FLOATS;
        const int first = st * PT;
        const bool have_next = st + 1 < stage_count;
        if (st == 0)
        {
            if (have_next)
            {
                run_stage(no, yes, stage, stage_next, first);
            }
            else
            {
                run_stage(no, no, stage, stage_next, first);
            }
        }
        else if (have_next)
        {
            run_stage(yes, yes, stage, stage_next, first);
        }
        else
        {
            run_stage(yes, no, stage, stage_next, first);
        }
        lds_barrier();
    }
    // the results of the last stage are still in the LDS tile
    static_for<0, NE>([&](auto e_tag) { store_rows(e_tag, read_rows(e_tag), (stage_count - 1) * PT); });
}

template <int DP>
bool launch_resident(int dim, size_t q, size_t n, const float* queries, size_t qs, const float* points,
                     size_t ps, float* dist, size_t ds, hipStream_t stream)
{
    using P = resident_geometry<DP>;
    size_t q_full = 0;
    size_t n_full = 0;
    if constexpr (DP <= 128)
    {
        // the pipelined kernel takes whole query blocks x whole stages when rows are 16-byte
        // aligned and every offset inside a workgroup's share fits the 32-bit buffer offsets
        using F = pipelined_geometry<DP>;
        const bool aligned = reinterpret_cast<std::uintptr_t>(dist) % 16 == 0 && ds % 4 == 0;
        const bool in_range = 32 * ds * sizeof(float) < (1ULL << 31) &&
                              static_cast<size_t>(dim) * ps * sizeof(float) < (1ULL << 31);
        if (aligned && in_range)
        {
            q_full = q / F::QB * F::QB;
            n_full = n / F::PT * F::PT;
            if (q_full == 0 || n_full == 0)
            {
                q_full = 0;
                n_full = 0;
            }
        }
        if (q_full > 0)
        {
            // One workgroup fits a compute unit (LDS), so its prologue and epilogue are not
            // overlapped with anything: give every workgroup as long a range of points as still
            // leaves about 8 workgroups per compute unit, at least 4096 points.
            const size_t gx = q_full / F::QB;
            size_t range = n_full * gx / 2048;
            range = range < 4096 ? 4096 : (range > (1U << 20) ? (1U << 20) : range);
            range = (range + F::PT - 1) / F::PT * F::PT;
            const size_t gy = (n_full + range - 1) / range;
            if (gx > 0x7FFFFFFFULL || gy > 65535)
            {
                return false;
            }
            hipLaunchKernelGGL((dist_pipelined_kernel<DP>), dim3(static_cast<unsigned>(gx), static_cast<unsigned>(gy)),
                               dim3(256), 0, stream, dim, q_full, n_full, queries, qs, points, ps, dist, ds,
                               static_cast<unsigned>(range));
        }
    }
    // the plain kernel covers what is left: points n_full.. of the first q_full queries, and all
    // points of the queries q_full..
    auto plain = [&](size_t q_first, size_t q_end, size_t n_first) -> bool {
        if (q_first >= q_end || n_first >= n)
        {
            return true;
        }
        const size_t gx = (q_end - q_first + P::QB - 1) / P::QB;
        const size_t gy = (n - n_first + P::RANGE - 1) / P::RANGE;
        if (gx > 0x7FFFFFFFULL || gy > 65535)
        {
            return false;
        }
        const dim3 grid(static_cast<unsigned>(gx), static_cast<unsigned>(gy));
        if (reinterpret_cast<std::uintptr_t>(dist) % 128 == 0 && ds % 32 == 0)
        {
            hipLaunchKernelGGL((dist_resident_kernel<DP, true>), grid, dim3(256), 0, stream, dim, q_end, n, queries,
                               qs, points, ps, dist, ds, q_first, n_first);
        }
        else
        {
            hipLaunchKernelGGL((dist_resident_kernel<DP, false>), grid, dim3(256), 0, stream, dim, q_end, n, queries,
                               qs, points, ps, dist, ds, q_first, n_first);
        }
        return true;
    };
    return plain(0, q_full, n_full) && plain(q_full, q, 0);
}

// Vectors given one after the other (component t of vector v at in[v * in_stride + t]) into the
// dim-major form the distance kernels read (out[t * out_stride + v]): 32 x 32 tiles through LDS, so
// that both sides are accessed in runs of consecutive addresses.
__global__ void __launch_bounds__(256) to_dim_major_kernel(const float* __restrict__ in, size_t in_stride,
                                                           float* __restrict__ out, size_t out_stride,
                                                           size_t count, int dim)
{
    __shared__ float tile[32][33];
    const int tx = static_cast<int>(threadIdx.x) & 31;
    const int ty = static_cast<int>(threadIdx.x) >> 5; // 0 .. 7
    const size_t v0 = static_cast<size_t>(blockIdx.x) * 32;
    const int t0 = static_cast<int>(blockIdx.y) * 32;
#pragma unroll
    for (int i = 0; i < 4; ++i)
    {
        const size_t v = v0 + ty + 8 * i;
        const int t = t0 + tx;
        tile[ty + 8 * i][tx] = v < count && t < dim ? in[v * in_stride + t] : 0.0F;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i)
    {
        const int t = t0 + ty + 8 * i;
        const size_t v = v0 + tx;
        if (t < dim && v < count)
        {
            out[static_cast<size_t>(t) * out_stride + v] = tile[tx][ty + 8 * i];
        }
    }
}

// row stride of a dim-major copy in the workspace: the count rounded up to whole 16-byte pieces
size_t padded_count(size_t count) { return (count + 3) / 4 * 4; }

} // namespace
} // namespace bitsknn

extern "C" size_t bitsknn_dist_layout_workspace_bytes(int dim, size_t q, size_t n, int queries_layout,
                                                      int points_layout)
{
    using namespace bitsknn;
    if (dim <= 0)
    {
        return 0;
    }
    size_t floats = 0;
    if (queries_layout == BITSKNN_LAYOUT_ROW_MAJOR)
    {
        floats += static_cast<size_t>(dim) * padded_count(q);
    }
    if (points_layout == BITSKNN_LAYOUT_ROW_MAJOR)
    {
        floats += static_cast<size_t>(dim) * padded_count(n);
    }
    return floats * sizeof(float);
}

extern "C" int bitsknn_dist_layout_f32(int op, int dim, size_t q, size_t n, const float* queries,
                                       int queries_layout, size_t query_stride, const float* points,
                                       int points_layout, size_t point_stride, float* dist,
                                       size_t dist_row_stride, void* workspace, size_t workspace_bytes,
                                       void* stream)
{
    using namespace bitsknn;
    clear_error();
    for (const int layout : {queries_layout, points_layout})
    {
        if (layout != BITSKNN_LAYOUT_ROW_MAJOR && layout != BITSKNN_LAYOUT_COLUMN_MAJOR)
        {
            return fail(BITSKNN_ERR_INVALID, "bitsknn_dist_layout_f32: unknown layout %d", layout);
        }
    }
    if (dim <= 0)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_dist_f32: dimension must be positive, got %d", dim);
    }
    if (q == 0 || n == 0)
    {
        return BITSKNN_OK;
    }
    if (queries == nullptr || points == nullptr)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_dist_f32: null pointer");
    }
    const size_t need = bitsknn_dist_layout_workspace_bytes(dim, q, n, queries_layout, points_layout);
    if (need != 0 && (workspace == nullptr || workspace_bytes < need ||
                      reinterpret_cast<std::uintptr_t>(workspace) % 16 != 0))
    {
        return fail(BITSKNN_ERR_INVALID,
                    "bitsknn_dist_layout_f32: vectors given one after the other need a 16-byte aligned workspace of "
                    "%zu bytes (bitsknn_dist_layout_workspace_bytes), got %zu",
                    need, workspace_bytes);
    }
    auto* hip_stream = static_cast<hipStream_t>(stream);
    auto* next = static_cast<float*>(workspace);
    // the dim-major operand of the kernels: the caller's array as it is, or its copy in the workspace
    auto dim_major = [&](const float*& base, int layout, size_t& stride, size_t count) -> int {
        if (layout == BITSKNN_LAYOUT_COLUMN_MAJOR)
        {
            return BITSKNN_OK;
        }
        if (stride < static_cast<size_t>(dim))
        {
            return fail(BITSKNN_ERR_INVALID, "bitsknn_dist_layout_f32: stride smaller than the dimension");
        }
        const size_t tiles = (count + 31) / 32;
        if (tiles > 0x7FFFFFFFULL || (dim + 31) / 32 > 65535)
        {
            return fail(BITSKNN_ERR_INVALID, "bitsknn_dist_layout_f32: too many vectors for one launch: %zu", count);
        }
        const size_t out_stride = padded_count(count);
        hipLaunchKernelGGL(to_dim_major_kernel, dim3(static_cast<unsigned>(tiles), static_cast<unsigned>((dim + 31) / 32)),
                           dim3(256), 0, hip_stream, base, stride, next, out_stride, count, dim);
        BITSKNN_HIP_CHECK(hipGetLastError());
        base = next;
        stride = out_stride;
        next += static_cast<size_t>(dim) * out_stride;
        return BITSKNN_OK;
    };
    int status = dim_major(queries, queries_layout, query_stride, q);
    if (status != BITSKNN_OK)
    {
        return status;
    }
    status = dim_major(points, points_layout, point_stride, n);
    if (status != BITSKNN_OK)
    {
        return status;
    }
    return bitsknn_dist_f32(op, dim, q, n, queries, query_stride, points, point_stride, dist, dist_row_stride, stream);
}

extern "C" int bitsknn_dist_f32(int op, int dim, size_t q, size_t n, const float* queries_dim_major,
                                size_t query_stride, const float* points_dim_major,
                                size_t point_stride, float* dist, size_t dist_row_stride, void* stream)
{
    using namespace bitsknn;
    clear_error();
    if (op != BITSKNN_DIST_L2 && op != BITSKNN_DIST_PARTIAL_L2 && op != BITSKNN_DIST_EXPANDED &&
        op != BITSKNN_DIST_PARTIAL_L2_BF16X3)
    {
        return fail(BITSKNN_ERR_UNSUPPORTED, "Unsupported distance: %d", op);
    }
    if (dim <= 0)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_dist_f32: dimension must be positive, got %d", dim);
    }
    if (q == 0 || n == 0)
    {
        return BITSKNN_OK;
    }
    if (queries_dim_major == nullptr || points_dim_major == nullptr || dist == nullptr)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_dist_f32: null pointer");
    }
    if (query_stride < q || point_stride < n || dist_row_stride < n)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_dist_f32: stride smaller than the vector count");
    }
    auto* hip_stream = static_cast<hipStream_t>(stream);
    if (op == BITSKNN_DIST_L2)
    {
        const size_t gx = (n + L2_PT - 1) / L2_PT;
        const size_t gy = (q + L2_QT - 1) / L2_QT;
        if (gx > 0x7FFFFFFFULL || gy > 65535)
        {
            return fail(BITSKNN_ERR_INVALID, "bitsknn_dist_f32: matrix too large for one launch (%zu x %zu)", q, n);
        }
        const bool aligned = reinterpret_cast<std::uintptr_t>(points_dim_major) % 16 == 0 &&
                             point_stride % 4 == 0 &&
                             reinterpret_cast<std::uintptr_t>(dist) % 16 == 0 && dist_row_stride % 4 == 0;
        const dim3 grid(static_cast<unsigned>(gx), static_cast<unsigned>(gy));
        if (aligned)
        {
            hipLaunchKernelGGL(dist_l2_kernel<true>, grid, dim3(WAVE * L2_WAVES), 0, hip_stream, dim, q,
                               n, queries_dim_major, query_stride, points_dim_major, point_stride, dist,
                               dist_row_stride);
        }
        else
        {
            hipLaunchKernelGGL(dist_l2_kernel<false>, grid, dim3(WAVE * L2_WAVES), 0, hip_stream, dim, q,
                               n, queries_dim_major, query_stride, points_dim_major, point_stride, dist,
                               dist_row_stride);
        }
    }
    else
    {
        // bf16x3 products where that kernel applies (dimensions 9 .. 64, aligned rows), else the fp32
        // matrix instructions
        if (op == BITSKNN_DIST_PARTIAL_L2_BF16X3 &&
            launch_dist_split(dim, q, n, queries_dim_major, query_stride, points_dim_major, point_stride, dist,
                              dist_row_stride, hip_stream))
        {
            BITSKNN_HIP_CHECK(hipGetLastError());
            return BITSKNN_OK;
        }
        bool launched = false;
        if (dim <= 8)
        {
            launched = launch_resident<8>(dim, q, n, queries_dim_major, query_stride, points_dim_major,
                                          point_stride, dist, dist_row_stride, hip_stream);
        }
        else if (dim <= 16)
        {
            launched = launch_resident<16>(dim, q, n, queries_dim_major, query_stride, points_dim_major,
                                           point_stride, dist, dist_row_stride, hip_stream);
        }
        else if (dim <= 32)
        {
            launched = launch_resident<32>(dim, q, n, queries_dim_major, query_stride, points_dim_major,
                                           point_stride, dist, dist_row_stride, hip_stream);
        }
        else if (dim <= 64)
        {
            launched = launch_resident<64>(dim, q, n, queries_dim_major, query_stride, points_dim_major,
                                           point_stride, dist, dist_row_stride, hip_stream);
        }
        else if (dim <= 128)
        {
            launched = launch_resident<128>(dim, q, n, queries_dim_major, query_stride, points_dim_major,
                                            point_stride, dist, dist_row_stride, hip_stream);
        }
        if (launched)
        {
            BITSKNN_HIP_CHECK(hipGetLastError());
            return BITSKNN_OK;
        }
        // larger dimensions: the generic tiled kernel
        const size_t gx = (q + MM_TILE - 1) / MM_TILE;
        const size_t gy = (n + MM_TILE - 1) / MM_TILE;
        if (gx > 0x7FFFFFFFULL || gy > 65535)
        {
            return fail(BITSKNN_ERR_INVALID, "bitsknn_dist_f32: matrix too large for one launch (%zu x %zu)", q, n);
        }
        hipLaunchKernelGGL(dist_mfma_kernel, dim3(static_cast<unsigned>(gx), static_cast<unsigned>(gy)),
                           dim3(256), 0, hip_stream, dim, q, n, queries_dim_major, query_stride,
                           points_dim_major, point_stride, dist, dist_row_stride);
    }
    BITSKNN_HIP_CHECK(hipGetLastError());
    return BITSKNN_OK;
}
