// Instantiations of the bits top-k kernel for one workgroup size (BITSKNN_TOPK_BS = 128, 256 or
// 512, given on the command line) so that the three sizes compile in parallel.
#include "topk_bits_kernel.hpp"

#ifndef BITSKNN_TOPK_BS
#error "compile with -DBITSKNN_TOPK_BS=128|256|512"
#endif

namespace bitsknn
{
namespace
{

template <int BS, int IPT, int L, bool VEC, bool SQ = false>
void launch(const topk_args& a, size_t rows, hipStream_t stream)
{
    hipLaunchKernelGGL((bits_topk_kernel<BS, IPT, L, VEC, SQ>), dim3(static_cast<u32>(rows)), dim3(BS),
                       0, stream, a);
}

// rows cut into parts, selected and (with topk_args::done) reduced in one launch: compiled for the
// depths the prefetching variant uses (an even number of 16-byte loads per thread; 4-byte loads
// in one shape); false otherwise
template <int BS, int IPT>
bool launch_parts(int loads, bool vec, const topk_args& a, size_t rows, hipStream_t stream)
{
    if (!vec)
    {
        launch<BS, IPT, 2, false, true>(a, rows, stream);
        return true;
    }
    switch (loads)
    {
    case 2:
        launch<BS, IPT, 2, true, true>(a, rows, stream);
        return true;
    case 4:
        launch<BS, IPT, 4, true, true>(a, rows, stream);
        return true;
    case 6:
        launch<BS, IPT, 6, true, true>(a, rows, stream);
        return true;
    case 8:
        launch<BS, IPT, 8, true, true>(a, rows, stream);
        return true;
    default:
        return false;
    }
}

// loads = number of 16-byte loads each thread keeps in flight per iteration
template <int BS, int IPT>
void launch_variant(int loads, bool vec, const topk_args& a, size_t rows, hipStream_t stream)
{
    if (!vec)
    {
        // rows that do not start on a 16-byte boundary: 4-byte loads, one fixed shape
        launch<BS, IPT, 2, false>(a, rows, stream);
        return;
    }
    switch (loads)
    {
    case 1:
        launch<BS, IPT, 1, true>(a, rows, stream);
        break;
    case 2:
        launch<BS, IPT, 2, true>(a, rows, stream);
        break;
    case 3:
        launch<BS, IPT, 3, true>(a, rows, stream);
        break;
    case 4:
        launch<BS, IPT, 4, true>(a, rows, stream);
        break;
    case 6:
        launch<BS, IPT, 6, true>(a, rows, stream);
        break;
    default:
        launch<BS, IPT, 8, true>(a, rows, stream);
        break;
    }
}

template <int BS, int IPT>
bool launch_either(int loads, bool vec, const topk_args& a, size_t rows, hipStream_t stream)
{
    if (a.parts > 1)
    {
        return launch_parts<BS, IPT>(loads, vec, a, rows, stream);
    }
    launch_variant<BS, IPT>(loads, vec, a, rows, stream);
    return true;
}

template <int BS>
bool launch_ipt(int ipt, int loads, bool vec, const topk_args& a, size_t rows, hipStream_t stream)
{
    switch (ipt)
    {
    case 1:
        return launch_either<BS, 1>(loads, vec, a, rows, stream);
    case 2:
        return launch_either<BS, 2>(loads, vec, a, rows, stream);
    case 4:
        return launch_either<BS, 4>(loads, vec, a, rows, stream);
    case 8:
        if constexpr (BS <= 256)
        {
            return launch_either<BS, 8>(loads, vec, a, rows, stream);
        }
        return false;
    case 16:
        if constexpr (BS <= 128)
        {
            return launch_either<BS, 16>(loads, vec, a, rows, stream);
        }
        return false;
    default:
        return false;
    }
}



} // namespace

#define BITSKNN_CAT2(a, b) a##b
#define BITSKNN_CAT(a, b) BITSKNN_CAT2(a, b)

// returns false when the list length ipt*BS is not compiled for this workgroup size (or, for rows
// cut into parts, when the loads are not of a compiled form)
bool BITSKNN_CAT(launch_topk_bits_, BITSKNN_TOPK_BS)(int ipt, int loads, bool vec,
                                                     const topk_args& a, size_t rows,
                                                     hipStream_t stream)
{
    return launch_ipt<BITSKNN_TOPK_BS>(ipt, loads, vec, a, rows, stream);
}

} // namespace bitsknn
