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
