// Launcher of the distance kernel with bf16x3 products (dist_split.hip).
#ifndef BITSKNN_CSRC_DIST_SPLIT_HPP_
#define BITSKNN_CSRC_DIST_SPLIT_HPP_

#include "common.hpp"

namespace bitsknn
{

// ||p||^2 - 2 q.p for dimensions 33 .. 64 into a matrix whose rows start on 16-byte boundaries.
// Returns false (nothing launched) for anything else; a launch error is left for hipGetLastError.
bool launch_dist_split(int dim, size_t q, size_t n, const float* queries_dim_major, size_t query_stride,
                       const float* points_dim_major, size_t point_stride, float* dist, size_t dist_row_stride,
                       hipStream_t stream);

} // namespace bitsknn

#endif // BITSKNN_CSRC_DIST_SPLIT_HPP_
