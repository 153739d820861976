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

#include "common.hpp"

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

template <int DP>
__global__ void __launch_bounds__(256)
    dist_resident_kernel(int dim, size_t q, size_t n, const float* __restrict__ queries, size_t qs,
                         const float* __restrict__ points, size_t ps, float* __restrict__ dist, size_t ds)
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
    const size_t wave_q0 = static_cast<size_t>(blockIdx.x) * G::QB + static_cast<size_t>(wave) * 32 * QPW;
    const size_t j_begin = static_cast<size_t>(blockIdx.y) * G::RANGE;
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
                            __builtin_nontemporal_store(acc[a][r], dist + i * ds + j);
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

template <int DP>
bool launch_resident(int dim, size_t q, size_t n, const float* queries, size_t qs, const float* points,
                     size_t ps, float* dist, size_t ds, hipStream_t stream)
{
    using G = resident_geometry<DP>;
    const size_t gx = (q + G::QB - 1) / G::QB;
    const size_t gy = (n + G::RANGE - 1) / G::RANGE;
    if (gx > 0x7FFFFFFFULL || gy > 65535)
    {
        return false;
    }
    hipLaunchKernelGGL(dist_resident_kernel<DP>, dim3(static_cast<unsigned>(gx), static_cast<unsigned>(gy)),
                       dim3(256), 0, stream, dim, q, n, queries, qs, points, ps, dist, ds);
    return true;
}

} // namespace
} // namespace bitsknn

extern "C" int bitsknn_dist_f32(int op, int dim, size_t q, size_t n, const float* queries_dim_major,
                                size_t query_stride, const float* points_dim_major,
                                size_t point_stride, float* dist, size_t dist_row_stride, void* stream)
{
    using namespace bitsknn;
    clear_error();
    if (op != BITSKNN_DIST_L2 && op != BITSKNN_DIST_PARTIAL_L2 && op != BITSKNN_DIST_EXPANDED)
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
