// C-ABI entry points of bits-fused: parameter validation, the choice between the fused kernel, its
// point-split form and the two-pass form, and dispatch to the kernels instantiated per list length
// in fused_inst.hip.
#include <atomic>
#include <initializer_list>

#include "common.hpp"
#include "fused_args.hpp"

namespace bitsknn
{
namespace
{

// arithmetic of the products for 9 <= d <= 64 (bitsknn_fused_set_arithmetic)
std::atomic<int> g_arithmetic{BITSKNN_FUSED_FP32};

bool in_list(int v, std::initializer_list<int> values)
{
    for (const int x : values)
    {
        if (x == v)
        {
            return true;
        }
    }
    return false;
}

// Number of point ranges for a problem: enough workgroups for two per compute unit, ranges of at
// least 4096 points and a multiple of 256, at most 64 ranges.
int choose_splits(int q, int n)
{
    const int tiles = (q + FQ_QB - 1) / FQ_QB;
    int splits = 1;
    while (splits < 64 && tiles * splits < 512 && n / (splits * 2) >= 4096)
    {
        splits *= 2;
    }
    return splits;
}

// Long lists (k >= 128): the 32-slot buffers of the fused kernel make every merge pay for the whole
// list, and its time grows with k.  When the caller's workspace can hold the
// q x n distance matrix (at most 16 GiB), the entry point with a workspace therefore computes the
// matrix there with the MFMA distance kernel and selects with the bits kernel: two passes whose
// time does not depend on k.  The matrix never leaves the workspace.
constexpr int TWO_PASS_MIN_K = 128;
constexpr size_t TWO_PASS_MAX_BYTES = 16ULL << 30;

size_t two_pass_bytes(std::int32_t q, std::int32_t n, int k)
{
    const size_t bytes = static_cast<size_t>(q) * static_cast<size_t>(n) * sizeof(float);
    return k >= TWO_PASS_MIN_K && bytes <= TWO_PASS_MAX_BYTES ? bytes : 0;
}

int fused_impl(const float* queries_dim_major, const float* points_dim_major, int dim, std::int32_t q,
               std::int32_t n, float* out_dist, std::int32_t* out_label, int k, int query_reg,
               int db_reg, int dim_reg, int block_query_dim, int dim_mult, void* workspace,
               size_t workspace_bytes, bool use_workspace, void* stream)
{
    clear_error();
    // the reference's nested dispatch, outermost first (fused_cache_knn.cu:72-144); the tuning
    // parameters are validated like there although the MFMA tiling does not depend on them
    if (!in_list(query_reg, {2, 4, 8, 16}))
    {
        return fail(BITSKNN_ERR_UNSUPPORTED, "Unsupported queries_reg value: %d", query_reg);
    }
    if (!in_list(db_reg, {4, 8, 16}))
    {
        return fail(BITSKNN_ERR_UNSUPPORTED, "Unsupported db_reg value: %d", db_reg);
    }
    if (!in_list(dim_reg, {1, 2, 4}))
    {
        return fail(BITSKNN_ERR_UNSUPPORTED, "Unsupported dim_reg value: %d", dim_reg);
    }
    if (!in_list(block_query_dim, {1, 2, 4}))
    {
        return fail(BITSKNN_ERR_UNSUPPORTED, "Unsupported query_block_size value: %d", block_query_dim);
    }
    if (!in_list(dim_mult, {1, 2, 4}))
    {
        return fail(BITSKNN_ERR_UNSUPPORTED, "Unsupported dim_mult value: %d", dim_mult);
    }
    if (!in_list(k, {4, 8, 16, 32, 64, 128, 256}))
    {
        return fail(BITSKNN_ERR_UNSUPPORTED, "Unsupported k value: %d", k);
    }
    if (dim < dim_mult * dim_reg)
    {
        return fail(BITSKNN_ERR_UNSUPPORTED, "Dimension of vectors must not be lower than %d, but is %d",
                    dim_mult * dim_reg, dim);
    }
    if (dim > 256)
    {
        return fail(BITSKNN_ERR_UNSUPPORTED, "Unsupported dimension: %d (at most 256)", dim);
    }
    if (q <= 0)
    {
        return BITSKNN_OK;
    }
    if (n <= 0)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_fused_l2_topk_f32: no points");
    }
    if (queries_dim_major == nullptr || points_dim_major == nullptr || out_dist == nullptr ||
        out_label == nullptr)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_fused_l2_topk_f32: null pointer");
    }
    if (static_cast<size_t>(q) > 65535U * FQ_QB)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_fused_l2_topk_f32: too many queries: %d", q);
    }

    const size_t matrix_bytes = use_workspace ? two_pass_bytes(q, n, k) : 0;
    if (matrix_bytes != 0 && workspace != nullptr && workspace_bytes >= matrix_bytes &&
        reinterpret_cast<std::uintptr_t>(workspace) % 16 == 0)
    {
        auto* matrix = static_cast<float*>(workspace);
        const bool split = g_arithmetic.load(std::memory_order_relaxed) == BITSKNN_FUSED_BF16X3;
        const int status = bitsknn_dist_f32(split ? BITSKNN_DIST_PARTIAL_L2_BF16X3 : BITSKNN_DIST_PARTIAL_L2, dim, static_cast<size_t>(q),
                                            static_cast<size_t>(n), queries_dim_major, static_cast<size_t>(q),
                                            points_dim_major, static_cast<size_t>(n), matrix,
                                            static_cast<size_t>(n), stream);
        if (status != BITSKNN_OK)
        {
            return status;
        }
        return bitsknn_topk_bits_f32(matrix, static_cast<size_t>(n), nullptr, 0, nullptr, static_cast<size_t>(q),
                                     static_cast<size_t>(n), out_dist, out_label, static_cast<size_t>(k),
                                     static_cast<std::uint32_t>(k), 512, 3, 0,
                                     stream);
    }

    int splits = use_workspace ? choose_splits(q, n) : 1;
    const size_t pairs = static_cast<size_t>(q) * static_cast<size_t>(splits) * static_cast<size_t>(k);
    if (splits > 1 && (workspace == nullptr || workspace_bytes < pairs * 8))
    {
        return fail(BITSKNN_ERR_INVALID,
                    "bitsknn_fused_l2_topk_f32_ws: workspace of %zu bytes is too small, %zu needed",
                    workspace_bytes, pairs * 8);
    }
    fused_args a{queries_dim_major, points_dim_major, dim, q, n, out_dist, out_label, 1, 0};
    if (splits > 1)
    {
        // partial lists [q][splits][k] in the workspace: distances first, then labels
        a.out_dist = static_cast<float*>(workspace);
        a.out_label = reinterpret_cast<std::int32_t*>(a.out_dist + pairs);
        a.splits = splits;
    }
    a.split_points = ((n + splits - 1) / splits + 255) / 256 * 256;

    auto* hip_stream = static_cast<hipStream_t>(stream);
    const bool split = g_arithmetic.load(std::memory_order_relaxed) == BITSKNN_FUSED_BF16X3;
    hipError_t status = hipSuccess;
    switch (k)
    {
    case 4:
        status = launch_fused_k_4(a, split, hip_stream);
        break;
    case 8:
        status = launch_fused_k_8(a, split, hip_stream);
        break;
    case 16:
        status = launch_fused_k_16(a, split, hip_stream);
        break;
    case 32:
        status = launch_fused_k_32(a, split, hip_stream);
        break;
    case 64:
        status = launch_fused_k_64(a, split, hip_stream);
        break;
    case 128:
        status = launch_fused_k_128(a, split, hip_stream);
        break;
    default:
        status = launch_fused_k_256(a, split, hip_stream);
        break;
    }
    BITSKNN_HIP_CHECK(status);
    if (splits > 1)
    {
        // one bits pass over the splits*k candidates of every query, labels carried along
        const size_t cols = static_cast<size_t>(splits) * static_cast<size_t>(k);
        return bitsknn_topk_bits_f32(a.out_dist, cols, a.out_label, cols, nullptr, static_cast<size_t>(q),
                                     cols, out_dist, out_label, static_cast<size_t>(k),
                                     static_cast<std::uint32_t>(k), 128, 4, 0, stream);
    }
    return BITSKNN_OK;
}

} // namespace
} // namespace bitsknn

extern "C" int bitsknn_fused_l2_topk_f32(const float* queries_dim_major,
                                         const float* points_dim_major, int dim, int32_t q,
                                         int32_t n, float* out_dist, int32_t* out_label, int k,
                                         int query_reg, int db_reg, int dim_reg, int block_query_dim,
                                         int dim_mult, void* stream)
{
    return bitsknn::fused_impl(queries_dim_major, points_dim_major, dim, q, n, out_dist, out_label, k,
                               query_reg, db_reg, dim_reg, block_query_dim, dim_mult, nullptr, 0, false,
                               stream);
}

extern "C" int bitsknn_fused_set_arithmetic(int arithmetic)
{
    bitsknn::clear_error();
    if (arithmetic != BITSKNN_FUSED_FP32 && arithmetic != BITSKNN_FUSED_BF16X3)
    {
        return bitsknn::fail(BITSKNN_ERR_INVALID, "bitsknn_fused_set_arithmetic: unknown arithmetic %d", arithmetic);
    }
    bitsknn::g_arithmetic.store(arithmetic, std::memory_order_relaxed);
    return BITSKNN_OK;
}

extern "C" int bitsknn_fused_get_arithmetic(void)
{
    return bitsknn::g_arithmetic.load(std::memory_order_relaxed);
}

extern "C" size_t bitsknn_fused_workspace_bytes(int32_t q, int32_t n, int k)
{
    if (q <= 0 || n <= 0 || k <= 0)
    {
        return 0;
    }
    const size_t matrix_bytes = bitsknn::two_pass_bytes(q, n, k);
    if (matrix_bytes != 0)
    {
        return matrix_bytes;
    }
    const int splits = bitsknn::choose_splits(q, n);
    return splits > 1 ? static_cast<size_t>(q) * static_cast<size_t>(splits) * static_cast<size_t>(k) * 8 : 0;
}

extern "C" int bitsknn_fused_l2_topk_f32_ws(const float* queries_dim_major,
                                            const float* points_dim_major, int dim, int32_t q,
                                            int32_t n, float* out_dist, int32_t* out_label, int k,
                                            int query_reg, int db_reg, int dim_reg,
                                            int block_query_dim, int dim_mult, void* workspace,
                                            size_t workspace_bytes, void* stream)
{
    return bitsknn::fused_impl(queries_dim_major, points_dim_major, dim, q, n, out_dist, out_label, k,
                               query_reg, db_reg, dim_reg, block_query_dim, dim_mult, workspace,
                               workspace_bytes, true, stream);
}
