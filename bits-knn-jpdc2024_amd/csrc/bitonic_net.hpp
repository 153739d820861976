// Bitonic sorting networks over 64-bit keys held in registers, for gfx950 (wave64).
//
// N = BS*IPT keys live IPT per thread in blocked order (thread t owns sorted positions
// t*IPT .. t*IPT+IPT-1).  Exchange distances below IPT stay inside a thread, distances below
// 64 threads use cross-lane moves inside the wave, larger ones go through LDS.  The same
// templates serve a whole workgroup (BS = threads of the workgroup, t = thread index) and small
// aligned lane groups inside one wave (BS = lanes per group, t = lane index inside the group).
//
// Counterpart of the reference's register networks
// (include/bits/topk/bitonic_sort_regs.cuh:86-218, 246-370, 386-460 and
// include/bits/topk/bitonic_sort_warp.cuh:22-101), which are laid out for 32-wide warps.
#ifndef BITSKNN_CSRC_BITONIC_NET_HPP_
#define BITSKNN_CSRC_BITONIC_NET_HPP_

#include "common.hpp"

namespace bitsknn
{

__device__ __forceinline__ u64 lane_xor(u64 x, int mask)
{
    const u32 lo = static_cast<u32>(__shfl_xor(static_cast<int>(static_cast<u32>(x)), mask, WAVE));
    const u32 hi = static_cast<u32>(__shfl_xor(static_cast<int>(static_cast<u32>(x >> 32U)), mask, WAVE));
    return (static_cast<u64>(hi) << 32U) | lo;
}

// One compare-exchange layer of a bitonic network over N = BS*IPT keys held IPT per thread in
// blocked order (thread t owns sorted positions t*IPT .. t*IPT+IPT-1).  K2 is the size of the
// sequences being merged in this phase, J the exchange distance.  DESC flips the final order.
template <int BS, int IPT, int K2, int J, bool DESC>
__device__ __forceinline__ void net_step(u64 (&x)[IPT], u64* scratch, int t)
{
    constexpr int N = BS * IPT;
    if constexpr (J < IPT)
    {
        // both elements live in this thread
#pragma unroll
        for (int r = 0; r < IPT; ++r)
        {
            if ((r & J) == 0)
            {
                bool down = DESC;
                if constexpr (K2 < IPT)
                {
                    down = (((r & K2) != 0) != DESC);
                }
                else if constexpr (K2 < N)
                {
                    down = (((t & (K2 / IPT)) != 0) != DESC);
                }
                const u64 a = x[r];
                const u64 b = x[r | J];
                const bool sw = (b < a) != down;
                x[r] = sw ? b : a;
                x[r | J] = sw ? a : b;
            }
        }
    }
    else
    {
        constexpr int M = J / IPT; // partner thread = t ^ M
        bool down = DESC;
        if constexpr (K2 < N)
        {
            down = (((t & (K2 / IPT)) != 0) != DESC);
        }
        const bool keep_min = (((t & M) == 0) != down);
        if constexpr (M < WAVE)
        {
#pragma unroll
            for (int r = 0; r < IPT; ++r)
            {
                const u64 o = lane_xor(x[r], M);
                const bool take = (o < x[r]) == keep_min;
                x[r] = take ? o : x[r];
            }
        }
        else
        {
            // partner lives in another wave: exchange through LDS, striped so that neighbouring
            // lanes touch neighbouring 8-byte slots
            __syncthreads();
#pragma unroll
            for (int r = 0; r < IPT; ++r)
            {
                scratch[r * BS + t] = x[r];
            }
            __syncthreads();
#pragma unroll
            for (int r = 0; r < IPT; ++r)
            {
                const u64 o = scratch[r * BS + (t ^ M)];
                const bool take = (o < x[r]) == keep_min;
                x[r] = take ? o : x[r];
            }
        }
    }
}

template <int BS, int IPT, int K2, int J, bool DESC>
__device__ __forceinline__ void net_phase(u64 (&x)[IPT], u64* scratch, int t)
{
    net_step<BS, IPT, K2, J, DESC>(x, scratch, t);
    if constexpr (J > 1)
    {
        net_phase<BS, IPT, K2, J / 2, DESC>(x, scratch, t);
    }
}

// full bitonic sort: phases K2 = 2, 4, ..., N
template <int BS, int IPT, int K2, bool DESC>
__device__ __forceinline__ void net_sort(u64 (&x)[IPT], u64* scratch, int t)
{
    net_phase<BS, IPT, K2, K2 / 2, DESC>(x, scratch, t);
    if constexpr (K2 < BS * IPT)
    {
        net_sort<BS, IPT, K2 * 2, DESC>(x, scratch, t);
    }
}

} // namespace bitsknn

#endif // BITSKNN_CSRC_BITONIC_NET_HPP_
