// What the kernels with bf16x3 products share: an fp32 value is cut exactly into three bf16 pieces,
// and a product of two such values is the fp32 sum of six products of pieces on the bf16 matrix
// instructions (v_mfma_f32_32x32x16_bf16).
#ifndef BITSKNN_CSRC_BF16X3_HPP_
#define BITSKNN_CSRC_BF16X3_HPP_

#include <type_traits>

#include "common.hpp"

namespace bitsknn
{
namespace
{

// f(integral_constant<int, BEGIN>) ... f(integral_constant<int, END - 1>), expanded by the front end
template <int BEGIN, int END, typename F>
__device__ __forceinline__ void static_for(F&& f)
{
    if constexpr (BEGIN < END)
    {
        f(std::integral_constant<int, BEGIN>{});
        static_for<BEGIN + 1, END>(f);
    }
}


typedef float vfloat16 __attribute__((ext_vector_type(16)));
typedef float vfloat4 __attribute__((ext_vector_type(4)));
typedef u32 vuint4 __attribute__((ext_vector_type(4)));
typedef __bf16 vbf16x8 __attribute__((ext_vector_type(8)));

// x[i] = x1 + x2 + x3 exactly, each piece with at most 8 significant bits (a bf16): the upper
// halves of x, of x - x1 and of x - x1 - x2.  Piece c of values 2j and 2j+1 shares word j of pc.
__device__ __forceinline__ void split_bf16x3(const float (&x)[8], vuint4& p1, vuint4& p2, vuint4& p3)
{
    u32 b1[8];
    u32 b2[8];
    u32 b3[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
    {
        b1[i] = __builtin_bit_cast(u32, x[i]);
        const float r = x[i] - __builtin_bit_cast(float, b1[i] & 0xFFFF0000U);
        b2[i] = __builtin_bit_cast(u32, r);
        const float l = r - __builtin_bit_cast(float, b2[i] & 0xFFFF0000U);
        b3[i] = __builtin_bit_cast(u32, l);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
    {
        // bytes 3:2 of the odd value above bytes 3:2 of the even one
        p1[j] = __builtin_amdgcn_perm(b1[2 * j + 1], b1[2 * j], 0x07060302U);
        p2[j] = __builtin_amdgcn_perm(b2[2 * j + 1], b2[2 * j], 0x07060302U);
        p3[j] = __builtin_amdgcn_perm(b3[2 * j + 1], b3[2 * j], 0x07060302U);
    }
}

} // namespace
} // namespace bitsknn

#endif // BITSKNN_CSRC_BF16X3_HPP_
