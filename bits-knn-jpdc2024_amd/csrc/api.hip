// Error reporting, version and the two small utility kernels of the bitsknn C ABI.
#include "common.hpp"

#include <cstring>

namespace bitsknn
{
namespace
{

thread_local char g_error[512] = "";

__global__ void fill_kernel(float* __restrict__ dst, size_t count, float value)
{
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < count; i += stride)
    {
        dst[i] = value;
    }
}

__global__ void label_offsets_kernel(std::int32_t* __restrict__ offsets, size_t total, size_t parts,
                                     size_t cols_per_part)
{
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < total)
    {
        offsets[i] = static_cast<std::int32_t>((i % parts) * cols_per_part);
    }
}

typedef float vfloat4 __attribute__((ext_vector_type(4)));

// Plain streaming read with the row-to-workgroup mapping of the top-k kernels: 256 threads per
// row, two 16-byte non-temporal loads per thread in flight, a running minimum as the only work.
__global__ void __launch_bounds__(256) stream_read_kernel(const float* __restrict__ in, size_t stride,
                                                          u32 cols, float* __restrict__ row_min)
{
    __shared__ float partial[4];
    const float* __restrict__ row = in + static_cast<size_t>(blockIdx.x) * stride;
    const int t = static_cast<int>(threadIdx.x);
    constexpr u32 CHUNK = 256 * 4 * 2;
    float m = __builtin_inff();
    u32 c = 0;
    for (; c + CHUNK <= cols; c += CHUNK)
    {
        const vfloat4* p = reinterpret_cast<const vfloat4*>(row + c) + t;
        const vfloat4 x = __builtin_nontemporal_load(p);
        const vfloat4 y = __builtin_nontemporal_load(p + 256);
        m = fminf(m, fminf(fminf(fminf(x.x, x.y), fminf(x.z, x.w)), fminf(fminf(y.x, y.y), fminf(y.z, y.w))));
    }
    for (c += static_cast<u32>(t); c < cols; c += 256)
    {
        m = fminf(m, row[c]);
    }
#pragma unroll
    for (int offset = 32; offset > 0; offset /= 2)
    {
        m = fminf(m, __shfl_xor(m, offset));
    }
    if ((t & 63) == 0)
    {
        partial[t / 64] = m;
    }
    __syncthreads();
    if (t == 0)
    {
        row_min[blockIdx.x] = fminf(fminf(partial[0], partial[1]), fminf(partial[2], partial[3]));
    }
}

} // namespace

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    std::vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

void clear_error() { g_error[0] = '\0'; }

} // namespace bitsknn

extern "C" const char* bitsknn_last_error(void) { return bitsknn::g_error; }

extern "C" const char* bitsknn_version(void) { return "bitsknn 0.1 (gfx950)"; }

extern "C" int bitsknn_fill_f32(float* dst, size_t count, float value, void* stream)
{
    using namespace bitsknn;
    clear_error();
    if (count == 0)
    {
        return BITSKNN_OK;
    }
    if (dst == nullptr)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_fill_f32: null pointer");
    }
    const size_t blocks = (count + 255) / 256;
    const unsigned grid = static_cast<unsigned>(blocks < 65536 ? blocks : 65536);
    hipLaunchKernelGGL(fill_kernel, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream), dst,
                       count, value);
    BITSKNN_HIP_CHECK(hipGetLastError());
    return BITSKNN_OK;
}

extern "C" int bitsknn_label_offsets(int32_t* offsets, size_t rows, size_t parts,
                                     size_t cols_per_part, void* stream)
{
    using namespace bitsknn;
    clear_error();
    const size_t total = rows * parts;
    if (total == 0)
    {
        return BITSKNN_OK;
    }
    if (offsets == nullptr || parts == 0)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_label_offsets: null pointer or zero parts");
    }
    if ((parts - 1) * cols_per_part > 0x7FFFFFFFULL)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_label_offsets: offsets exceed int32");
    }
    const size_t blocks = (total + 255) / 256;
    if (blocks > 0x7FFFFFFFULL)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_label_offsets: too many rows");
    }
    hipLaunchKernelGGL(label_offsets_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), offsets, total, parts, cols_per_part);
    BITSKNN_HIP_CHECK(hipGetLastError());
    return BITSKNN_OK;
}

extern "C" int bitsknn_stream_read_f32(const float* in, size_t in_row_stride, size_t rows, size_t cols,
                                       float* row_min, void* stream)
{
    using namespace bitsknn;
    clear_error();
    if (rows == 0)
    {
        return BITSKNN_OK;
    }
    if (in == nullptr || row_min == nullptr)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_stream_read_f32: null pointer");
    }
    if (cols == 0 || cols > 0x7FFFFFFFULL || rows > 0x7FFFFFFFULL || in_row_stride < cols)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_stream_read_f32: bad matrix shape %zu x %zu (stride %zu)", rows,
                    cols, in_row_stride);
    }
    if (reinterpret_cast<std::uintptr_t>(in) % 16 != 0 || in_row_stride % 4 != 0)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_stream_read_f32: rows must start on 16-byte boundaries");
    }
    hipLaunchKernelGGL(stream_read_kernel, dim3(static_cast<unsigned>(rows)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), in, in_row_stride, static_cast<u32>(cols), row_min);
    BITSKNN_HIP_CHECK(hipGetLastError());
    return BITSKNN_OK;
}
