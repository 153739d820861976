// The stage image of the exact fused kernels: every stage of the point matrix as it stands in LDS
// (fp32 rows, cells of bf16 pieces, norm cells), one stage after the other in global memory, so
// that the fused kernel stages by copying instead of cutting the points again in every workgroup.
#include "fused_kernel.hpp"

namespace bitsknn
{
namespace
{

// One workgroup per stage: builds the stage in LDS the way the fused kernel's own staging does
// (same cut, same shares of the norm, points from n on with the norm that only passes an infinite
// radius) and copies it out.
template <int DP>
__global__ void __launch_bounds__(FQ_THREADS) fused_image_kernel(const float* points, int dim, int n, vuint4* image)
{
    using G = fused_geometry<DP, FUSED_ARITH_EXACT, 32>;
    constexpr int PT = G::PT;
    constexpr int VPT = G::VPT;
    constexpr int KS = G::KS;
    constexpr int STAGE_FLOATS = G::STAGE_FLOATS;
    __shared__ __attribute__((aligned(16))) float stage[STAGE_FLOATS];
    const int t = static_cast<int>(threadIdx.x);
    const int base = static_cast<int>(blockIdx.x) * PT;
    for (int i = t; i < STAGE_FLOATS; i += FQ_THREADS)
    {
        stage[i] = 0.0F;
    }
    __syncthreads();
    const int sp = t % PT;
    const int sd0 = VPT * (t / PT);
    const int norm_slot = DP == 64 ? t / WAVE : t / PT;
    const bool inside = base + sp < n;
    float eight[8];
    float share = 0.0F;
#pragma unroll
    for (int i = 0; i < 8; ++i)
    {
        const int dd = sd0 + i;
        eight[i] = 0.0F;
        if (i < VPT && dd < dim && inside)
        {
            eight[i] = points[static_cast<size_t>(dd) * static_cast<size_t>(n) + static_cast<size_t>(base + sp)];
        }
    }
    vuint4 piece[2];
    cut_bf16x2(eight, piece[0], piece[1]);
#pragma unroll
    for (int i = 0; i < VPT; ++i)
    {
        share = __builtin_fmaf(eight[i], eight[i], share);
        stage[(sd0 + i) * PT + sp] = eight[i];
    }
    constexpr int PIECE2 = DP <= 8 ? 1 : KS; // first cell of the second pieces
    if constexpr (VPT == 8)
    {
        vuint4* const cells = reinterpret_cast<vuint4*>(stage + DP * PT);
        cells[t] = piece[0];
        cells[PIECE2 * PT + t] = piece[1];
    }
    else
    {
        typedef u32 vuint2 __attribute__((ext_vector_type(2)));
        vuint2* const halves = reinterpret_cast<vuint2*>(stage + DP * PT);
        const int h = sd0 / 4;
        halves[2 * sp + h] = vuint2{piece[0][0], piece[0][1]};
        halves[2 * (PIECE2 * PT + sp) + h] = vuint2{piece[1][0], piece[1][1]};
    }
    if constexpr (DP == 64)
    {
        share += __builtin_bit_cast(float, lane_xor32<32>(__builtin_bit_cast(u32, share)));
    }
    {
        const float lowered = __builtin_fmaf(-NORM_LOWER, share, share);
        const vfloat2 whole{lowered, 0.0F};
        const u32 first = __builtin_bit_cast(u32, __builtin_convertvector(whole, vbf16x2)) & 0xFFFFU;
        const vfloat2 rest{lowered - __builtin_bit_cast(float, first << 16U), 0.0F};
        const u32 second = __builtin_bit_cast(u32, __builtin_convertvector(rest, vbf16x2)) & 0xFFFFU;
        u32* const norm_cell =
            reinterpret_cast<u32*>(reinterpret_cast<vuint4*>(stage + DP * PT) + (G::CELLS - 1) * PT + sp);
        norm_cell[norm_slot] = inside ? first | (second << 16U) : BF16_HUGE;
    }
    __syncthreads();
    vuint4* const out = image + static_cast<size_t>(blockIdx.x) * (STAGE_FLOATS / 4);
    for (int u = t; u < STAGE_FLOATS / 4; u += FQ_THREADS)
    {
        out[u] = reinterpret_cast<const vuint4*>(stage)[u];
    }
}

template <int DP>
constexpr size_t stage_bytes()
{
    return static_cast<size_t>(fused_geometry<DP, FUSED_ARITH_EXACT, 32>::STAGE_FLOATS) * sizeof(float);
}

template <int DP>
constexpr int stage_points()
{
    return fused_geometry<DP, FUSED_ARITH_EXACT, 32>::PT;
}

template <int DP>
hipError_t launch_image(const float* points, int dim, int n, void* image, hipStream_t stream)
{
    const unsigned stages = static_cast<unsigned>((n + stage_points<DP>() - 1) / stage_points<DP>());
    hipLaunchKernelGGL((fused_image_kernel<DP>), dim3(stages), dim3(FQ_THREADS), 0, stream, points, dim, n,
                       static_cast<vuint4*>(image));
    return hipGetLastError();
}

} // namespace

size_t fused_image_bytes(int dim, int n)
{
    if (dim < 1 || dim > 64 || n < 1)
    {
        return 0;
    }
    const size_t per_stage = dim <= 8 ? stage_bytes<8>() : dim <= 16 ? stage_bytes<16>() : dim <= 32 ? stage_bytes<32>() : stage_bytes<64>();
    const size_t points = dim <= 8 ? stage_points<8>() : dim <= 16 ? stage_points<16>() : dim <= 32 ? stage_points<32>() : stage_points<64>();
    return (static_cast<size_t>(n) + points - 1) / points * per_stage;
}

hipError_t launch_fused_image(const float* points, int dim, int n, void* image, hipStream_t stream)
{
    return dim <= 8    ? launch_image<8>(points, dim, n, image, stream)
           : dim <= 16 ? launch_image<16>(points, dim, n, image, stream)
           : dim <= 32 ? launch_image<32>(points, dim, n, image, stream)
                       : launch_image<64>(points, dim, n, image, stream);
}

} // namespace bitsknn
