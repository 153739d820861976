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

// split: the products of dimensions 9 .. 64 from three bf16 pieces per operand (below 9 the fp32
// matrix instructions are as fast)
hipError_t BITSKNN_CAT_EXPANDED(launch_fused_k_, BITSKNN_FUSED_K)(const fused_args& a, bool split,
                                                                  hipStream_t stream)
{
    constexpr int K = BITSKNN_FUSED_K;
    if (split && a.dim > 8 && a.dim <= 64)
    {
        return a.dim <= 16   ? launch_fused<K, 16, true>(a, stream)
               : a.dim <= 32 ? launch_fused<K, 32, true>(a, stream)
                             : launch_fused<K, 64, true>(a, stream);
    }
    if (a.dim <= 8)
    {
        return launch_fused<K, 8, false>(a, stream);
    }
    if (a.dim <= 16)
    {
        return launch_fused<K, 16, false>(a, stream);
    }
    if (a.dim <= 32)
    {
        return launch_fused<K, 32, false>(a, stream);
    }
    if (a.dim <= 64)
    {
        return launch_fused<K, 64, false>(a, stream);
    }
    if (a.dim <= 128)
    {
        return launch_fused<K, 128, false>(a, stream);
    }
    return launch_fused<K, 256, false>(a, stream);
}

} // namespace bitsknn
