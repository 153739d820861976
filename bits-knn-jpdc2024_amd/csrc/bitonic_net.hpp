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

// Value of `x` held by lane (lane ^ MASK), MASK a power of two below 64.  Distances 1, 2 and 8 are
// single data-parallel-primitive moves inside a row of 16 lanes (full VALU rate); 4 takes two
// masked row shifts, 16 and 32 a row / half-wave swap of gfx950 plus a select.
// XBAR: bit set of the distances that go through the LDS crossbar instead (ds_swizzle /
// ds_bpermute, no memory access).  That takes instructions off the vector ALU at the price of
// LDS latency: it pays where a merge is an occasional, vector-ALU-bound burst (bits top-k at
// large k: +1 % at k = 512, +2.4 % at k = 2048 on 1024 x 2^20 rows) and costs where all waves
// sort all the time (partial-bitonic-regs: -15 % at k = 32).
constexpr int XBAR_NONE = 0;
constexpr int XBAR_4_16_32 = 4 | 16 | 32;

template <int MASK, int XBAR = XBAR_NONE>
__device__ __forceinline__ u32 lane_xor32(u32 x)
{
    static_assert(MASK == 1 || MASK == 2 || MASK == 4 || MASK == 8 || MASK == 16 || MASK == 32);
    const int v = static_cast<int>(x);
    if constexpr ((XBAR & MASK) != 0 && MASK < 32)
    {
        // bit-mask mode: lane' = (lane & 0x1F) ^ MASK inside each half-wave
        return static_cast<u32>(__builtin_amdgcn_ds_swizzle(v, 0x1F | (MASK << 10)));
    }
    else if constexpr ((XBAR & MASK) != 0)
    {
        return static_cast<u32>(__builtin_amdgcn_ds_bpermute(static_cast<int>((threadIdx.x ^ 32U) << 2U), v));
    }
    else if constexpr (MASK == 1)
    {
        return static_cast<u32>(__builtin_amdgcn_mov_dpp(v, 0xB1, 0xF, 0xF, false)); // quad_perm [1,0,3,2]
    }
    else if constexpr (MASK == 2)
    {
        return static_cast<u32>(__builtin_amdgcn_mov_dpp(v, 0x4E, 0xF, 0xF, false)); // quad_perm [2,3,0,1]
    }
    else if constexpr (MASK == 4)
    {
        // lanes 0-3 and 8-11 of a row read 4 lanes up (row_shl:4), the others 4 lanes down
        const int up = __builtin_amdgcn_update_dpp(v, v, 0x104, 0xF, 0x5, false);
        return static_cast<u32>(__builtin_amdgcn_update_dpp(up, v, 0x114, 0xF, 0xA, false));
    }
    else if constexpr (MASK == 8)
    {
        return static_cast<u32>(__builtin_amdgcn_mov_dpp(v, 0x128, 0xF, 0xF, false)); // row_ror:8
    }
    else if constexpr (MASK == 16)
    {
        // swaps the odd 16-lane rows of the first copy with the even rows of the second
        const auto swapped = __builtin_amdgcn_permlane16_swap(x, x, false, false);
        return (threadIdx.x & 16U) != 0 ? swapped[0] : swapped[1];
    }
    else
    {
        const auto swapped = __builtin_amdgcn_permlane32_swap(x, x, false, false);
        return (threadIdx.x & 32U) != 0 ? swapped[0] : swapped[1];
    }
}

template <int MASK, int XBAR = XBAR_NONE>
__device__ __forceinline__ u64 lane_xor(u64 x)
{
    const u32 lo = lane_xor32<MASK, XBAR>(static_cast<u32>(x));
    const u32 hi = lane_xor32<MASK, XBAR>(static_cast<u32>(x >> 32U));
    return (static_cast<u64>(hi) << 32U) | lo;
}

// Whether bit X (a power of two) of the thread index `t` is set, as a per-lane predicate.  The
// lane index is t % 64, so below 64 the answer is a constant lane mask that costs no vector
// instruction; from 64 on it is the same for the whole wave.
template <int X>
__device__ __forceinline__ bool thread_bit(int t)
{
    static_assert(X > 0 && (X & (X - 1)) == 0);
    if constexpr (X == 1)
    {
        return __builtin_amdgcn_inverse_ballot_w64(0xAAAAAAAAAAAAAAAAULL);
    }
    else if constexpr (X == 2)
    {
        return __builtin_amdgcn_inverse_ballot_w64(0xCCCCCCCCCCCCCCCCULL);
    }
    else if constexpr (X == 4)
    {
        return __builtin_amdgcn_inverse_ballot_w64(0xF0F0F0F0F0F0F0F0ULL);
    }
    else if constexpr (X == 8)
    {
        return __builtin_amdgcn_inverse_ballot_w64(0xFF00FF00FF00FF00ULL);
    }
    else if constexpr (X == 16)
    {
        return __builtin_amdgcn_inverse_ballot_w64(0xFFFF0000FFFF0000ULL);
    }
    else if constexpr (X == 32)
    {
        return __builtin_amdgcn_inverse_ballot_w64(0xFFFFFFFF00000000ULL);
    }
    else
    {
        return (__builtin_amdgcn_readfirstlane(t) & X) != 0;
    }
}

// One compare-exchange layer of a bitonic network over N = BS*IPT keys held IPT per thread in
// blocked order (thread t owns sorted positions t*IPT .. t*IPT+IPT-1).  K2 is the size of the
// sequences being merged in this phase, J the exchange distance.  DESC flips the final order.
// `t` must be the thread index whose low 6 bits are the lane index.
// PP: `scratch` has room for 2N keys and consecutive LDS exchanges alternate between its halves
// (`flip`, the same in every thread), which saves the barrier that otherwise protects the readers
// of one exchange from the writers of the next.
template <int BS, int IPT, int K2, int J, bool DESC, int XBAR = XBAR_NONE, bool PP = false>
__device__ __forceinline__ void net_step(u64 (&x)[IPT], u64* scratch, int t, int& flip)
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
                    down = thread_bit<K2 / IPT>(t) != DESC;
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
            down = thread_bit<K2 / IPT>(t) != DESC;
        }
        const bool keep_min = thread_bit<M>(t) == down; // lower thread of the pair keeps the minimum when ascending
        if constexpr (M < WAVE)
        {
#pragma unroll
            for (int r = 0; r < IPT; ++r)
            {
                const u64 o = lane_xor<M, XBAR>(x[r]);
                const bool take = (o < x[r]) == keep_min;
                x[r] = take ? o : x[r];
            }
        }
        else
        {
            // partner lives in another wave: exchange through LDS, striped so that neighbouring
            // lanes touch neighbouring 8-byte slots
            u64* half = scratch;
            if constexpr (PP)
            {
                half = scratch + (flip != 0 ? N : 0);
                flip ^= 1;
            }
            else
            {
                __syncthreads();
            }
#pragma unroll
            for (int r = 0; r < IPT; ++r)
            {
                half[r * BS + t] = x[r];
            }
            __syncthreads();
#pragma unroll
            for (int r = 0; r < IPT; ++r)
            {
                const u64 o = half[r * BS + (t ^ M)];
                const bool take = (o < x[r]) == keep_min;
                x[r] = take ? o : x[r];
            }
        }
    }
}

template <int BS, int IPT, int K2, int J, bool DESC, int XBAR = XBAR_NONE, bool PP = false>
__device__ __forceinline__ void net_phase(u64 (&x)[IPT], u64* scratch, int t, int& flip)
{
    net_step<BS, IPT, K2, J, DESC, XBAR, PP>(x, scratch, t, flip);
    if constexpr (J > 1)
    {
        net_phase<BS, IPT, K2, J / 2, DESC, XBAR, PP>(x, scratch, t, flip);
    }
}

// full bitonic sort: phases K2 = 2, 4, ..., N
template <int BS, int IPT, int K2, bool DESC, int XBAR = XBAR_NONE, bool PP = false>
__device__ __forceinline__ void net_sort(u64 (&x)[IPT], u64* scratch, int t, int& flip)
{
    net_phase<BS, IPT, K2, K2 / 2, DESC, XBAR, PP>(x, scratch, t, flip);
    if constexpr (K2 < BS * IPT)
    {
        net_sort<BS, IPT, K2 * 2, DESC, XBAR, PP>(x, scratch, t, flip);
    }
}

// single-buffer forms (two barriers per LDS exchange)
template <int BS, int IPT, int K2, int J, bool DESC>
__device__ __forceinline__ void net_phase(u64 (&x)[IPT], u64* scratch, int t)
{
    int unused = 0;
    net_phase<BS, IPT, K2, J, DESC, XBAR_NONE, false>(x, scratch, t, unused);
}

template <int BS, int IPT, int K2, bool DESC>
__device__ __forceinline__ void net_sort(u64 (&x)[IPT], u64* scratch, int t)
{
    int unused = 0;
    net_sort<BS, IPT, K2, DESC, XBAR_NONE, false>(x, scratch, t, unused);
}

} // namespace bitsknn

#endif // BITSKNN_CSRC_BITONIC_NET_HPP_
