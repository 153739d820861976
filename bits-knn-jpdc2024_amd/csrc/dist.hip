// Distance kernels (placeholder until implemented).
#include "common.hpp"

extern "C" int bitsknn_dist_f32(int, int, size_t, size_t, const float*, size_t, const float*, size_t,
                                float*, size_t, void*)
{
    return bitsknn::fail(BITSKNN_ERR_UNSUPPORTED, "bitsknn_dist_f32: not implemented");
}
