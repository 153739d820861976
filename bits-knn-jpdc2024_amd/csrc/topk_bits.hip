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
                      out_row_stride, k, 1, nullptr, nullptr, nullptr, 0};
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

extern "C" int bitsknn_topk_bits_parts_f32(const float* in, size_t rows, size_t cols, uint32_t parts,
                                           float* part_dist, int32_t* part_label, int32_t* counters,
                                           float* out_dist, int32_t* out_label, size_t out_row_stride,
                                           uint32_t k, uint32_t block_size, uint32_t items_per_thread,
                                           void* stream)
{
    using namespace bitsknn;
    if (parts <= 1)
    {
        return bitsknn_topk_bits_f32(in, cols, nullptr, 0, nullptr, rows, cols, out_dist, out_label,
                                     out_row_stride, k, block_size, items_per_thread, 1, stream);
    }
    clear_error();
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
    if (in == nullptr || out_dist == nullptr || out_label == nullptr || part_dist == nullptr ||
        part_label == nullptr || counters == nullptr)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_topk_bits_parts_f32: null pointer");
    }
    if (cols == 0 || cols > 0x7FFFFFFFULL || cols % parts != 0)
    {
        return fail(BITSKNN_ERR_INVALID,
                    "bitsknn_topk_bits_parts_f32: cols must be in [1, 2^31-1] and a multiple of the parts, got %zu "
                    "and %u parts",
                    cols, parts);
    }
    if (rows * parts > 0x7FFFFFFFULL || static_cast<size_t>(parts) * k > 0x7FFFFFFFULL)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_topk_bits_parts_f32: too many rows or parts: %zu x %u", rows, parts);
    }
    if (out_row_stride < k)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_topk_bits_parts_f32: row stride smaller than row length");
    }
    u32 compiled_k = 16;
    while (compiled_k < k)
    {
        compiled_k *= 2;
    }
    const int ipt = compiled_k <= block_size ? 1 : static_cast<int>(compiled_k / block_size);
    // always the prefetching form, as the reference's bits-sq (bits_knn.cu:137)
    const int loads = static_cast<int>((items_per_thread + 3) / 4) * 2;
    const size_t part_cols = cols / parts;
    const bool vec = (reinterpret_cast<std::uintptr_t>(in) % 16 == 0) && (part_cols % 4 == 0);
    // The second pass reads the parts' pairs with the loads of the first: with 16-byte loads every
    // logical row's pairs have to start on a 16-byte boundary.  Otherwise it is a launch of its own.
    // One launch pays up to about four workgroups per compute unit: the reduction of a row then starts
    // while other rows are still streaming.  With more parts in flight than that all rows end together
    // and a second launch, which the runtime starts behind the first without a gap, is as fast or
    // faster (64 rows of 2^19 values, k = 16: 16 parts 36.2 us in one launch, 36.9 us in two; 32 parts
    // 44.2 / 37.2 us; 256 rows, 8 parts: 100 / 92 us).
    const size_t merged = static_cast<size_t>(parts) * k;
    const bool one_launch = rows * parts <= 1024 &&
                            (!vec || (merged % 4 == 0 && reinterpret_cast<std::uintptr_t>(part_dist) % 16 == 0));
    const topk_args a{in,        part_cols, nullptr,   0,         nullptr,  static_cast<u32>(part_cols),
                      part_dist, part_label, k,        k,         parts,    one_launch ? counters : nullptr,
                      out_dist,  out_label, out_row_stride};
    auto* hip_stream = static_cast<hipStream_t>(stream);
    bool ok = false;
    switch (block_size)
    {
    case 128:
        ok = launch_topk_bits_128(ipt, loads, vec, a, rows * parts, hip_stream);
        break;
    case 256:
        ok = launch_topk_bits_256(ipt, loads, vec, a, rows * parts, hip_stream);
        break;
    default:
        ok = launch_topk_bits_512(ipt, loads, vec, a, rows * parts, hip_stream);
        break;
    }
    if (!ok)
    {
        return fail(BITSKNN_ERR_UNSUPPORTED, "Unsupported k value: %u", k);
    }
    BITSKNN_HIP_CHECK(hipGetLastError());
    if (!one_launch)
    {
        return bitsknn_topk_bits_f32(part_dist, merged, part_label, merged, nullptr, rows, merged, out_dist,
                                     out_label, out_row_stride, k, block_size, items_per_thread, 1, stream);
    }
    return BITSKNN_OK;
}
