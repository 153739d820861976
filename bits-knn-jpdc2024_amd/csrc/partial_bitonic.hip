// partial-bitonic-regs for gfx950: top-k by repeated sort-and-merge in registers, without any
// filtering of the input.  Every value of a row goes through a sorting network, which makes this
// kernel the "no buffer" baseline against which the bits kernel's filter and buffer are measured.
//
// Replaces the reference's partial_bitonic_regs_kernel and its dispatch
// (src/topk/singlepass/partial_bitonic.cu:217-294, 341-358): the row is consumed in blocks of
// BS*IPT values, IPT = ceil(K / BS); each block is sorted descending, the element-wise minimum
// with the ascending list of the best BS*IPT values so far is a bitonic sequence holding the
// new best values, and one merge phase sorts it again.
//
// One workgroup per row; the keys are the 64-bit (value, label) keys of the bits kernel, so
// equal values come out by lower label.  The values of the next block are requested from HBM
// before the current block is sorted.

#include "bitonic_net.hpp"
#include "common.hpp"

namespace bitsknn
{
namespace
{

struct partial_args
{
    const float* in;
    size_t in_stride;
    u32 cols;
    float* out_dist;
    std::int32_t* out_label;
    size_t out_stride;
    u32 k;
};

template <int BS, int IPT>
__global__ void __launch_bounds__(BS) partial_bitonic_kernel(const partial_args a)
{
    constexpr int N = BS * IPT;
    // exchange scratch for distances of 64 lanes and more (none in a single-wave workgroup)
    __shared__ u64 scratch[BS > WAVE ? N : 1];

    const int t = static_cast<int>(threadIdx.x);
    const float* __restrict__ row = a.in + static_cast<size_t>(blockIdx.x) * a.in_stride;
    const u32 n = a.cols;

    // value r of this thread in the block that starts at `base` is column base + r*BS + t
    auto fetch = [&](float (&v)[IPT], u32 base) {
#pragma unroll
        for (int r = 0; r < IPT; ++r)
        {
            const u32 col = base + static_cast<u32>(r * BS + t);
            v[r] = col < n ? row[col] : __builtin_inff();
        }
    };
    auto to_keys = [&](u64 (&x)[IPT], const float (&v)[IPT], u32 base) {
#pragma unroll
        for (int r = 0; r < IPT; ++r)
        {
            const u32 col = base + static_cast<u32>(r * BS + t);
            x[r] = col < n ? make_key(v[r], static_cast<std::int32_t>(col)) : PAD_KEY;
        }
    };

    float v[IPT];
    u64 best[IPT];
    fetch(v, 0);
    to_keys(best, v, 0);
    if (static_cast<u32>(N) < n)
    {
        fetch(v, N);
    }
    net_sort<BS, IPT, 2, false>(best, scratch, t);

    for (u32 base = N; base < n; base += N)
    {
        u64 next[IPT];
        to_keys(next, v, base);
        if (base + N < n)
        {
            fetch(v, base + N);
        }
        net_sort<BS, IPT, 2, true>(next, scratch, t);
#pragma unroll
        for (int r = 0; r < IPT; ++r)
        {
            best[r] = next[r] < best[r] ? next[r] : best[r];
        }
        net_phase<BS, IPT, N, N / 2, false>(best, scratch, t);
    }

    float* __restrict__ out_d = a.out_dist + static_cast<size_t>(blockIdx.x) * a.out_stride;
    std::int32_t* __restrict__ out_l = a.out_label + static_cast<size_t>(blockIdx.x) * a.out_stride;
#pragma unroll
    for (int r = 0; r < IPT; ++r)
    {
        const u32 e = static_cast<u32>(t * IPT + r);
        if (e < a.k)
        {
            out_d[e] = key_value(best[r]);
            out_l[e] = key_label(best[r]);
        }
    }
}

template <int BS, int IPT>
void launch(const partial_args& a, size_t rows, hipStream_t stream)
{
    hipLaunchKernelGGL((partial_bitonic_kernel<BS, IPT>), dim3(static_cast<unsigned>(rows)), dim3(BS), 0,
                       stream, a);
}

template <int BS>
bool launch_block(int ipt, const partial_args& a, size_t rows, hipStream_t stream)
{
    switch (ipt)
    {
    case 1:
        launch<BS, 1>(a, rows, stream);
        return true;
    case 2:
        launch<BS, 2>(a, rows, stream);
        return true;
    case 4:
        launch<BS, 4>(a, rows, stream);
        return true;
    case 8:
        if constexpr (BS <= 256)
        {
            launch<BS, 8>(a, rows, stream);
            return true;
        }
        return false;
    case 16:
        if constexpr (BS <= 128)
        {
            launch<BS, 16>(a, rows, stream);
            return true;
        }
        return false;
    case 32:
        if constexpr (BS <= 64)
        {
            launch<BS, 32>(a, rows, stream);
            return true;
        }
        return false;
    default:
        return false;
    }
}

} // namespace
} // namespace bitsknn

extern "C" int bitsknn_topk_partial_bitonic_f32(const float* in, size_t in_row_stride, size_t rows,
                                                size_t cols, float* out_dist, int32_t* out_label,
                                                size_t out_row_stride, uint32_t k, uint32_t block_size,
                                                void* stream)
{
    using namespace bitsknn;
    clear_error();
    // block sizes and k values of the reference's dispatch (partial_bitonic.cu:345-357)
    if (block_size != 64 && block_size != 128 && block_size != 256 && block_size != 512)
    {
        return fail(BITSKNN_ERR_UNSUPPORTED, "Unsupported block size: %u", block_size);
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
        return fail(BITSKNN_ERR_INVALID, "bitsknn_topk_partial_bitonic_f32: null matrix pointer");
    }
    if (cols == 0 || cols > 0x7FFFFFFFULL - 2 * 2048)
    {
        return fail(BITSKNN_ERR_INVALID,
                    "bitsknn_topk_partial_bitonic_f32: cols must be in [1, 2^31-4097], got %zu", cols);
    }
    if (rows > 0x7FFFFFFFULL)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_topk_partial_bitonic_f32: too many rows: %zu", rows);
    }
    if (in_row_stride < cols || out_row_stride < k)
    {
        return fail(BITSKNN_ERR_INVALID,
                    "bitsknn_topk_partial_bitonic_f32: row stride smaller than row length");
    }
    u32 compiled_k = 16;
    while (compiled_k < k)
    {
        compiled_k *= 2;
    }
    const int ipt = static_cast<int>((compiled_k + block_size - 1) / block_size);
    const partial_args a{in, in_row_stride, static_cast<u32>(cols), out_dist, out_label, out_row_stride, k};
    auto* hip_stream = static_cast<hipStream_t>(stream);
    bool ok = false;
    switch (block_size)
    {
    case 64:
        ok = launch_block<64>(ipt, a, rows, hip_stream);
        break;
    case 128:
        ok = launch_block<128>(ipt, a, rows, hip_stream);
        break;
    case 256:
        ok = launch_block<256>(ipt, a, rows, hip_stream);
        break;
    default:
        ok = launch_block<512>(ipt, a, rows, hip_stream);
        break;
    }
    if (!ok)
    {
        return fail(BITSKNN_ERR_UNSUPPORTED, "Unsupported k value: %u", k);
    }
    BITSKNN_HIP_CHECK(hipGetLastError());
    return BITSKNN_OK;
}
