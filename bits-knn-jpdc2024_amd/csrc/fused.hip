// Fused distance + top-k kernel (placeholder until implemented).
#include "common.hpp"

extern "C" int bitsknn_fused_l2_topk_f32(const float*, const float*, int, int32_t, int32_t, float*,
                                         int32_t*, int, int, int, int, int, int, void*)
{
    return bitsknn::fail(BITSKNN_ERR_UNSUPPORTED, "bitsknn_fused_l2_topk_f32: not implemented");
}
