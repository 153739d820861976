// C-ABI entry point of the bits top-k selection: parameter validation and dispatch to the
// kernels instantiated per workgroup size in topk_bits_inst.hip.
#include "topk_bits_kernel.hpp"

namespace bitsknn
{
bool launch_topk_bits_128(int ipt, int loads, bool vec, const topk_args& a, size_t rows,
                          hipStream_t stream);
bool launch_topk_bits_256(int ipt, int loads, bool vec, const topk_args& a, size_t rows,
                          hipStream_t stream);
bool launch_topk_bits_512(int ipt, int loads, bool vec, const topk_args& a, size_t rows,
                          hipStream_t stream);
} // namespace bitsknn

extern "C" int bitsknn_topk_bits_f32(const float* in, size_t in_row_stride, const int32_t* in_label,
                                     size_t label_row_stride, const int32_t* label_offsets,
                                     size_t rows, size_t cols, float* out_dist, int32_t* out_label,
                                     size_t out_row_stride, uint32_t k, uint32_t block_size,
                                     uint32_t items_per_thread, int prefetch, void* stream)
{
    using namespace bitsknn;
    clear_error();
    // parameter lists of the reference build (definitions_all.hpp:4-5, definitions_common.hpp:4),
    // checked in the order of its nested dispatch (bits_knn.cu:40-62)
    if (block_size != 128 && block_size != 256 && block_size != 512)
    {
        return fail(BITSKNN_ERR_UNSUPPORTED, "Unsupported block size: %u", block_size);
    }
    if (items_per_thread < 1 || items_per_thread > 16)
    {
        return fail(BITSKNN_ERR_UNSUPPORTED, "Unsupported batch size: %u", items_per_thread);
    }
    if (k < 1 || k > 2048)
    {
        return fail(BITSKNN_ERR_UNSUPPORTED, "Unsupported k value: %u", k);
    }
    if (rows == 0)
    {
        return BITSKNN_OK;
    }
    if (in == nullptr || out_dist == nullptr || out_label == nullptr)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_topk_bits_f32: null matrix pointer");
    }
    if (cols == 0 || cols > 0x7FFFFFFFULL)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_topk_bits_f32: cols must be in [1, 2^31-1], got %zu",
                    cols);
    }
    if (rows > 0x7FFFFFFFULL)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_topk_bits_f32: too many rows: %zu", rows);
    }
    if (in_row_stride < cols || out_row_stride < k || (in_label != nullptr && label_row_stride < cols))
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_topk_bits_f32: row stride smaller than row length");
    }

    u32 compiled_k = 16;
    while (compiled_k < k)
    {
        compiled_k *= 2;
    }
    const int ipt = compiled_k <= block_size ? 1 : static_cast<int>(compiled_k / block_size);
    // values in flight per thread: the batch size rounded up to whole 16-byte loads, doubled for
    // the prefetching variant
    const int loads = static_cast<int>((items_per_thread + 3) / 4) * (prefetch != 0 ? 2 : 1);
    // 16-byte loads need every row to start on a 16-byte boundary
    const bool vec = (reinterpret_cast<std::uintptr_t>(in) % 16 == 0) && (in_row_stride % 4 == 0);

    const topk_args a{in,      in_row_stride, in_label,  label_row_stride,
                      label_offsets, static_cast<u32>(cols), out_dist, out_label,
                      out_row_stride, k};
    auto* hip_stream = static_cast<hipStream_t>(stream);
    bool ok = false;
    switch (block_size)
    {
    case 128:
        ok = launch_topk_bits_128(ipt, loads, vec, a, rows, hip_stream);
        break;
    case 256:
        ok = launch_topk_bits_256(ipt, loads, vec, a, rows, hip_stream);
        break;
    default:
        ok = launch_topk_bits_512(ipt, loads, vec, a, rows, hip_stream);
        break;
    }
    if (!ok)
    {
        return fail(BITSKNN_ERR_UNSUPPORTED, "Unsupported k value: %u", k);
    }
    BITSKNN_HIP_CHECK(hipGetLastError());
    return BITSKNN_OK;
}
