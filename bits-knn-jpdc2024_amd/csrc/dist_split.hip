// Partial squared L2 distance matrix (||p||^2 - 2 q.p) with bf16x3 products, for gfx950, dimensions
// 33 .. 64: BITSKNN_DIST_PARTIAL_L2_BF16X3 of bitsknn_dist_f32.  (Up to 32 dimensions the fp32 kernel
// is bound by the stores of the matrix already, and faster at them.)
//
// Same result layout and the same role as the fp32 kernel of dist.hip (the reference's
// partial_l2_ops, include/bits/distance/abstract_gemm.cuh:108-170); the products run on the bf16
// matrix instructions, which leaves the kernel bound by the stores of the matrix instead of by the
// fp32 matrix unit:
//
//  * A workgroup of 4 waves owns 128 queries (32 per wave), whose three bf16 pieces of -2q stay in
//    registers as B operands, and a range of points, walked in stages of 64 or 128 points, two
//    stages in LDS (one multiplied, one filled; one barrier per stage).
//  * The staging threads cut the points into pieces: per piece and 8 dimensions one 16-byte cell
//    per point (the A operand of v_mfma_f32_32x32x16_bf16), then the norms, which the accumulators
//    start from.
//  * A 32 x 32 result tile (a lane holds 16 distances of one query) goes through a per-wave LDS
//    tile so that every store instruction writes whole 128-byte lines of 8 matrix rows.

#include "bf16x3.hpp"
#include "bitonic_net.hpp"
#include "common.hpp"
#include "dist_split.hpp"

namespace bitsknn
{
namespace
{

constexpr int DS_THREADS = 256;
constexpr int DS_QB = 128;            // queries per workgroup
constexpr int DS_TILE_STRIDE = 36;    // floats per query row of the result tile in LDS (32 + padding)

template <int DK>
struct dist_split_geometry
{
    static constexpr int KB = DK / 16;                   // matrix steps of 16 dimensions
    static constexpr int KS = DK / 8;                    // cells of 8 dimensions per point and piece
    static constexpr int PT = DK <= 16 ? 128 : 64;       // points per stage
    static constexpr int CPT = KS * PT / DS_THREADS;     // cells a staging thread cuts per stage
    static constexpr int TPP = KS / CPT;                 // staging threads per point (neighbouring lanes)
    static constexpr int MT = PT / 32;                   // row tiles per stage
    static constexpr int STAGE_FLOATS = 3 * KS * PT * 4 + PT;
    static_assert(CPT >= 1 && TPP * CPT == KS && (TPP == 2 || TPP == 4));
    static constexpr size_t lds_bytes()
    {
        return (2 * static_cast<size_t>(STAGE_FLOATS) + 4 * 32 * DS_TILE_STRIDE) * sizeof(float);
    }
};

struct dist_split_args
{
    int dim;
    size_t q;
    size_t n;
    const float* queries; // dim-major
    size_t query_stride;
    const float* points;  // dim-major
    size_t point_stride;
    float* dist;          // row-major q x n, rows 16-byte aligned
    size_t dist_stride;
    unsigned range;       // points per blockIdx.y, a multiple of the stage
};

template <int DK>
__global__ void __launch_bounds__(DS_THREADS) dist_split_kernel(const dist_split_args a)
{
    using G = dist_split_geometry<DK>;
    constexpr int KB = G::KB;
    constexpr int KS = G::KS;
    constexpr int PT = G::PT;
    constexpr int CPT = G::CPT;
    constexpr int TPP = G::TPP;
    constexpr int MT = G::MT;
    constexpr int STAGE_FLOATS = G::STAGE_FLOATS;

    extern __shared__ float lds[];
    float* const stages = lds;                                   // [2][STAGE_FLOATS]
    float* const tiles = lds + 2 * STAGE_FLOATS;                 // [waves][32][DS_TILE_STRIDE]

    const int t = static_cast<int>(threadIdx.x);
    const int lane = t & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(t / WAVE);
    const int half = lane / 32;
    const int ql = lane & 31;
    const size_t wave_q0 = static_cast<size_t>(blockIdx.x) * DS_QB + static_cast<size_t>(wave) * 32;
    const size_t my_q = wave_q0 + ql;
    const size_t n_begin = static_cast<size_t>(blockIdx.y) * a.range;
    const size_t n_end = n_begin + a.range < a.n ? n_begin + a.range : a.n;
    float* const tile = tiles + wave * 32 * DS_TILE_STRIDE;

    // the three pieces of -2q for the 8 dimensions 16*kb + 8*half .. + 7 of step kb
    vuint4 qs[3][KB];
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
    {
        float val[8];
#pragma unroll
        for (int j = 0; j < 8; ++j)
        {
            const int dd = 16 * kb + 8 * half + j;
            val[j] = 0.0F;
            if (dd < a.dim && my_q < a.q)
            {
                val[j] = -2.0F * a.queries[static_cast<size_t>(dd) * a.query_stride + my_q];
            }
        }
        split_bf16x3(val, qs[0][kb], qs[1][kb], qs[2][kb]);
    }

    // staging: thread t cuts cells ks0 .. ks0+CPT-1 (8 dimensions each) of point t / TPP
    const int sp = t / TPP;
    const int ks0 = (t % TPP) * CPT;
    // Point values are read with buffer loads: a constant byte offset per value and lane (beyond the
    // resource for dimensions from dim on, which then read as zero; the hardware checks the lane
    // offset only) plus the scalar offset of the stage, so that a load needs no vector arithmetic.
    float pre[CPT][8];
    const auto point_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(a.points), 0, static_cast<int>(static_cast<size_t>(a.dim) * a.point_stride * sizeof(float)),
        0x00020000);
    constexpr int OUTSIDE = 0x7FFFFFF0;
    int load_off[CPT][8];
#pragma unroll
    for (int c = 0; c < CPT; ++c)
    {
#pragma unroll
        for (int i = 0; i < 8; ++i)
        {
            const int dd = 8 * (ks0 + c) + i;
            load_off[c][i] = dd < a.dim ? static_cast<int>((static_cast<size_t>(dd) * a.point_stride + sp) * sizeof(float))
                                        : OUTSIDE;
        }
    }
    auto fetch = [&](size_t base) __attribute__((always_inline)) {
        const int stage_off = static_cast<int>(base * sizeof(float));
        // ragged last stage of the range: points from its end on read as zero
        const bool inside = base + PT <= n_end || base + sp < n_end;
#pragma unroll
        for (int c = 0; c < CPT; ++c)
        {
#pragma unroll
            for (int i = 0; i < 8; ++i)
            {
                pre[c][i] = __builtin_bit_cast(
                    float, __builtin_amdgcn_raw_buffer_load_b32(point_rsrc, inside ? load_off[c][i] : OUTSIDE,
                                                                stage_off, 0));
            }
        }
    };
    auto deposit = [&](float* stage, size_t base) __attribute__((always_inline)) {
        vuint4* const cells = reinterpret_cast<vuint4*>(stage);
        float share = 0.0F;
#pragma unroll
        for (int c = 0; c < CPT; ++c)
        {
#pragma unroll
            for (int i = 0; i < 8; ++i)
            {
                share = __builtin_fmaf(pre[c][i], pre[c][i], share);
            }
            vuint4 piece[3];
            split_bf16x3(pre[c], piece[0], piece[1], piece[2]);
#pragma unroll
            for (int p = 0; p < 3; ++p)
            {
                cells[(p * KS + ks0 + c) * PT + sp] = piece[p];
            }
        }
        share += __builtin_bit_cast(float, lane_xor32<1>(__builtin_bit_cast(u32, share)));
        if constexpr (TPP == 4)
        {
            share += __builtin_bit_cast(float, lane_xor32<2>(__builtin_bit_cast(u32, share)));
        }
        (void)base;
        stage[3 * KS * PT * 4 + sp] = share;
    };

    // The wave's 32 rows of the matrix as a buffer: rows from q on lie beyond it and are dropped by
    // the hardware; a store is a constant lane offset (row, 16-byte chunk) plus the scalar offset of
    // the tile's first column.
    const size_t wave_rows = wave_q0 < a.q ? (a.q - wave_q0 < 32 ? a.q - wave_q0 : 32) : 0;
    const auto out_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        a.dist + wave_q0 * a.dist_stride, 0, static_cast<int>(wave_rows * a.dist_stride * sizeof(float)), 0x00020000);
    int store_off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
    {
        const int idx = j * WAVE + lane;
        store_off[j] = static_cast<int>((static_cast<size_t>(idx / 8) * a.dist_stride + 4 * (idx % 8)) * sizeof(float));
    }

    // one 32 x 32 tile: through the wave's LDS tile to whole lines of the matrix
    auto store_tile = [&](const vfloat16& acc, size_t col_base) __attribute__((always_inline)) {
#pragma unroll
        for (int g = 0; g < 4; ++g)
        {
            const vfloat4 v = {acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]};
            *reinterpret_cast<vfloat4*>(tile + ql * DS_TILE_STRIDE + 8 * g + 4 * half) = v;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const int tile_off = static_cast<int>(col_base * sizeof(float));
        const bool whole = col_base + 32 <= n_end; // wave-uniform
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            const int idx = j * WAVE + lane;
            const int row = idx / 8;
            const int chunk = idx % 8;
            const vuint4 v = *reinterpret_cast<const vuint4*>(tile + row * DS_TILE_STRIDE + 4 * chunk);
            if (whole)
            {
                __builtin_amdgcn_raw_buffer_store_b128(v, out_rsrc, store_off[j], tile_off, 2);
            }
            else
            {
                // ragged end of the range: whole chunks while they fit, then single values
                const size_t col = col_base + 4 * chunk;
                if (col + 4 <= n_end)
                {
                    __builtin_amdgcn_raw_buffer_store_b128(v, out_rsrc, store_off[j], tile_off, 2);
                }
                else
                {
#pragma unroll
                    for (int e = 0; e < 3; ++e)
                    {
                        if (col + e < n_end)
                        {
                            __builtin_amdgcn_raw_buffer_store_b32(v[e], out_rsrc,
                                                                  store_off[j] + e * static_cast<int>(sizeof(float)),
                                                                  tile_off, 0);
                        }
                    }
                }
            }
        }
        // the next tile is written by the same wave after its reads above
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };

    auto multiply = [&](const float* stage, size_t base) __attribute__((always_inline)) {
        const vuint4* const cells = reinterpret_cast<const vuint4*>(stage);
        const float* const norm_row = stage + 3 * KS * PT * 4;
        // the six products of a step, smallest terms first
        constexpr int order[6][2] = {{2, 0}, {1, 1}, {0, 2}, {1, 0}, {0, 1}, {0, 0}};
        static_for<0, MT / 2>([&](auto p_tag) {
            constexpr int p = decltype(p_tag)::value;
            vuint4 af[2][3][KB];
#pragma unroll
            for (int tl = 0; tl < 2; ++tl)
            {
#pragma unroll
                for (int c = 0; c < 3; ++c)
                {
#pragma unroll
                    for (int kb = 0; kb < KB; ++kb)
                    {
                        af[tl][c][kb] = cells[(c * KS + 2 * kb + half) * PT + p * 64 + tl * 32 + ql];
                    }
                }
            }
            vfloat16 acc0;
            vfloat16 acc1;
            const float* norms = norm_row + p * 64 + 4 * half;
#pragma unroll
            for (int g = 0; g < 4; ++g)
            {
                const vfloat4 x = *reinterpret_cast<const vfloat4*>(norms + 8 * g);
                const vfloat4 y = *reinterpret_cast<const vfloat4*>(norms + 32 + 8 * g);
#pragma unroll
                for (int e = 0; e < 4; ++e)
                {
                    acc0[4 * g + e] = x[e];
                    acc1[4 * g + e] = y[e];
                }
            }
            static_for<0, KB>([&](auto kb_tag) {
                constexpr int kb = decltype(kb_tag)::value;
                static_for<0, 6>([&](auto o_tag) {
                    constexpr int ca = order[decltype(o_tag)::value][0];
                    constexpr int cb = order[decltype(o_tag)::value][1];
                    acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                        __builtin_bit_cast(vbf16x8, af[0][ca][kb]), __builtin_bit_cast(vbf16x8, qs[cb][kb]), acc0,
                        0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                        __builtin_bit_cast(vbf16x8, af[1][ca][kb]), __builtin_bit_cast(vbf16x8, qs[cb][kb]), acc1,
                        0, 0, 0);
                });
            });
            store_tile(acc0, base + p * 64);
            store_tile(acc1, base + p * 64 + 32);
        });
    };

    fetch(n_begin);
    deposit(stages, n_begin);
    if (n_begin + PT < n_end)
    {
        fetch(n_begin + PT);
    }
    __syncthreads();
    int parity = 0;
    for (size_t base = n_begin; base < n_end; base += PT)
    {
        multiply(stages + parity * STAGE_FLOATS, base);
        parity ^= 1;
        if (base + PT < n_end)
        {
            deposit(stages + parity * STAGE_FLOATS, base + PT);
            if (base + 2 * PT < n_end)
            {
                fetch(base + 2 * PT);
            }
        }
        __syncthreads();
    }
}

template <int DK>
bool launch(const dist_split_args& args, hipStream_t stream)
{
    using G = dist_split_geometry<DK>;
    constexpr size_t lds_bytes = G::lds_bytes();
    if (lds_bytes > 48 * 1024)
    {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(&dist_split_kernel<DK>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)) != hipSuccess)
        {
            return false;
        }
    }
    dist_split_args a = args;
    // ranges of 16,384 points (whole stages), longer when the grid would not hold them
    size_t range = 16384;
    while ((a.n + range - 1) / range > 65535)
    {
        range *= 2;
    }
    if (range > 0x80000000ULL)
    {
        return false;
    }
    a.range = static_cast<unsigned>(range);
    const size_t gx = (a.q + DS_QB - 1) / DS_QB;
    const size_t gy = (a.n + range - 1) / range;
    if (gx > 0x7FFFFFFFULL)
    {
        return false;
    }
    hipLaunchKernelGGL((dist_split_kernel<DK>), dim3(static_cast<unsigned>(gx), static_cast<unsigned>(gy)),
                       dim3(DS_THREADS), lds_bytes, stream, a);
    return true;
}

} // namespace

bool launch_dist_split(int dim, size_t q, size_t n, const float* queries_dim_major, size_t query_stride,
                       const float* points_dim_major, size_t point_stride, float* dist, size_t dist_row_stride,
                       hipStream_t stream)
{
    if (dim <= 32 || dim > 64 || reinterpret_cast<std::uintptr_t>(dist) % 16 != 0 || dist_row_stride % 4 != 0)
    {
        return false;
    }
    // the kernel addresses the points and a wave's 32 matrix rows with 32-bit buffer offsets
    if (static_cast<size_t>(dim) * point_stride * sizeof(float) >= (1ULL << 31) ||
        32 * dist_row_stride * sizeof(float) >= (1ULL << 31) || n * sizeof(float) >= (1ULL << 31))
    {
        return false;
    }
    const dist_split_args args{dim,  q,           n, queries_dim_major, query_stride, points_dim_major, point_stride,
                               dist, dist_row_stride, 0};
    return launch<64>(args, stream);
}

} // namespace bitsknn
