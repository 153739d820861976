// Shared host/device helpers of the bitsknn HIP library (gfx950, wave64).
#ifndef BITSKNN_CSRC_COMMON_HPP_
#define BITSKNN_CSRC_COMMON_HPP_

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "bitsknn.h"

namespace bitsknn
{

using u32 = std::uint32_t;
using u64 = unsigned long long;

constexpr int WAVE = 64;

// ---- error reporting ------------------------------------------------------------------------

// Stores a printf-formatted message for bitsknn_last_error() and returns `code`.
int fail(int code, const char* fmt, ...);
void clear_error();

#define BITSKNN_HIP_CHECK(expr)                                                                   \
    do                                                                                            \
    {                                                                                             \
        const hipError_t status_ = (expr);                                                        \
        if (status_ != hipSuccess)                                                                \
        {                                                                                         \
            return ::bitsknn::fail(BITSKNN_ERR_HIP, "%s:%d %s: %s", __FILE__, __LINE__,           \
                                   hipGetErrorName(status_), hipGetErrorString(status_));         \
        }                                                                                         \
    } while (0)

// ---- order-preserving 64-bit keys ----------------------------------------------------------
//
// A (value, label) pair is held as one unsigned 64-bit key whose integer order is the
// lexicographic order (value ascending as IEEE floats, then label ascending as int32).  A
// sorting network over such keys is a total order, so equal values always come out by lower
// label.  -0.0 is folded onto +0.0 (they compare equal as floats); a NaN of either sign takes the
// key of +inf, so that every path treats it as +inf (and writes it back as +inf).

__host__ __device__ __forceinline__ u32 float_key(float v)
{
    union
    {
        float f;
        u32 u;
    } c;
    c.f = fminf(v + 0.0F, __builtin_inff()); // -0.0 -> +0.0, NaN -> +inf
    const u32 b = c.u;
    return b ^ (static_cast<u32>(static_cast<std::int32_t>(b) >> 31) | 0x80000000U);
}

__host__ __device__ __forceinline__ float key_float(u32 k)
{
    union
    {
        float f;
        u32 u;
    } c;
    c.u = (k & 0x80000000U) != 0 ? (k ^ 0x80000000U) : ~k;
    return c.f;
}

__host__ __device__ __forceinline__ u64 make_key(float v, std::int32_t label)
{
    return (static_cast<u64>(float_key(v)) << 32U) |
           static_cast<u64>(static_cast<u32>(label) ^ 0x80000000U);
}

__host__ __device__ __forceinline__ float key_value(u64 key)
{
    return key_float(static_cast<u32>(key >> 32U));
}

__host__ __device__ __forceinline__ std::int32_t key_label(u64 key)
{
    return static_cast<std::int32_t>(static_cast<u32>(key) ^ 0x80000000U);
}

// (+inf, INT32_MAX): sorts after every finite value and after real +inf entries
constexpr u64 PAD_KEY = 0xFF800000FFFFFFFFULL;

// Workgroup barrier that orders LDS traffic only, so that global loads issued earlier stay in
// flight across it.
__device__ __forceinline__ void lds_barrier()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

} // namespace bitsknn

#endif // BITSKNN_CSRC_COMMON_HPP_
