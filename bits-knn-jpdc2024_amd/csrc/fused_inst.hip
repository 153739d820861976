// Instantiations of the bits-fused kernel for one list length (BITSKNN_FUSED_K = 4 ... 256, given
// on the command line) so that the list lengths compile in parallel.
#include "fused_kernel.hpp"

#ifndef BITSKNN_FUSED_K
#error "compile with -DBITSKNN_FUSED_K=4|8|16|32|64|128|256"
#endif

namespace bitsknn
{

#define BITSKNN_CAT2(a, b) a##b
#define BITSKNN_CAT(a, b) a##b
#define BITSKNN_CAT_EXPANDED(a, b) BITSKNN_CAT2(a, b)

// FUSED_ARITH_BF16X3: dimensions 9 .. 64 (below 9 the fp32 matrix instructions are as fast);
// FUSED_ARITH_EXACT: dimensions up to 128 (a stage holds the points twice, as fp32 rows and as bf16
// pieces; 65 .. 128 dimensions only in workgroups of 256 queries, whatever fused_args::workgroup
// says; 129 .. 256 with the fp32 matrix instructions as the filter); everything else takes the fp32
// matrix instructions
hipError_t BITSKNN_CAT_EXPANDED(launch_fused_k_, BITSKNN_FUSED_K)(const fused_args& a, int arith,
                                                                  hipStream_t stream)
{
    constexpr int K = BITSKNN_FUSED_K;
    if (arith == FUSED_ARITH_BF16X3 && a.dim > 8 && a.dim <= 64)
    {
        return a.dim <= 16   ? launch_fused<K, 16, FUSED_ARITH_BF16X3>(a, stream)
               : a.dim <= 32 ? launch_fused<K, 32, FUSED_ARITH_BF16X3>(a, stream)
                             : launch_fused<K, 64, FUSED_ARITH_BF16X3>(a, stream);
    }
    if (arith == FUSED_ARITH_EXACT && a.dim <= 64)
    {
        return a.dim <= 8    ? launch_fused<K, 8, FUSED_ARITH_EXACT>(a, stream)
               : a.dim <= 16 ? launch_fused<K, 16, FUSED_ARITH_EXACT>(a, stream)
               : a.dim <= 32 ? launch_fused<K, 32, FUSED_ARITH_EXACT>(a, stream)
                             : launch_fused<K, 64, FUSED_ARITH_EXACT>(a, stream);
    }
    if (arith == FUSED_ARITH_EXACT && a.dim <= 128)
    {
        return launch_fused_as<K, 128, FUSED_ARITH_EXACT, false, true>(a, stream);
    }
    if (arith == FUSED_ARITH_EXACT)
    {
        // 129 .. 256 dimensions: the fp32 matrix instructions as the filter
        return launch_fused<K, 256, FUSED_ARITH_EXACT_F32>(a, stream);
    }
    if (a.dim <= 8)
    {
        return launch_fused<K, 8, FUSED_ARITH_MFMA_F32>(a, stream);
    }
    if (a.dim <= 16)
    {
        return launch_fused<K, 16, FUSED_ARITH_MFMA_F32>(a, stream);
    }
    if (a.dim <= 32)
    {
        return launch_fused<K, 32, FUSED_ARITH_MFMA_F32>(a, stream);
    }
    if (a.dim <= 64)
    {
        return launch_fused<K, 64, FUSED_ARITH_MFMA_F32>(a, stream);
    }
    if (a.dim <= 128)
    {
        return launch_fused<K, 128, FUSED_ARITH_MFMA_F32>(a, stream);
    }
    return launch_fused<K, 256, FUSED_ARITH_MFMA_F32>(a, stream);
}

} // namespace bitsknn
