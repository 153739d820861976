// Test-only kernels that drive the register sorting networks of csrc/bitonic_net.hpp directly
// (built into tests/libnettest.so by the package Makefile; loaded by tests/test_networks_gpu.py).
//
// Counterpart of the reference's direct network test (tests/bitonic_sort_regs_test.cu:21-160:
// block_sort over (items per thread, block size) pairs, ascending and descending).
#include <hip/hip_runtime.h>

#include "bitonic_net.hpp"

namespace
{
using bitsknn::u64;

// OP 0: full sort (net_sort).  OP 1: the last merge phase only (net_phase with K2 = N, J = N/2),
// which sorts a bitonic sequence.
// BS >= 64: one group of N = BS*IPT keys per workgroup of BS threads, LDS exchanges for distances
// of 64 lanes and more (PP: two alternating LDS regions).  BS < 64: 64/BS groups per wave, each in
// an aligned range of BS lanes, no LDS (the form the fused kernel uses for its per-query buffers).
template <int BS, int IPT, int XBAR, bool PP, bool DESC, int OP>
__global__ void __launch_bounds__(BS < 64 ? 64 : BS) net_kernel(u64* data)
{
    constexpr int N = BS * IPT;
    constexpr int THREADS = BS < 64 ? 64 : BS;
    constexpr int GROUPS = THREADS / BS;
    __shared__ u64 scratch[BS >= 128 ? (PP ? 2 * N : N) : 1];
    const int thread = static_cast<int>(threadIdx.x);
    const int t = thread % BS;
    u64* const group = data + (static_cast<size_t>(blockIdx.x) * GROUPS + thread / BS) * N;
    u64 x[IPT];
#pragma unroll
    for (int r = 0; r < IPT; ++r)
    {
        x[r] = group[t * IPT + r];
    }
    int flip = 0;
    if constexpr (OP == 0)
    {
        bitsknn::net_sort<BS, IPT, 2, DESC, XBAR, PP>(x, scratch, t, flip);
    }
    else
    {
        bitsknn::net_phase<BS, IPT, N, N / 2, DESC, XBAR, PP>(x, scratch, t, flip);
    }
#pragma unroll
    for (int r = 0; r < IPT; ++r)
    {
        group[t * IPT + r] = x[r];
    }
}

template <int BS, int IPT, int XBAR, bool PP, bool DESC>
int launch(int op, u64* data, int groups, hipStream_t stream)
{
    constexpr int THREADS = BS < 64 ? 64 : BS;
    constexpr int GROUPS = THREADS / BS;
    if (groups % GROUPS != 0)
    {
        return 2;
    }
    if (op == 0)
    {
        hipLaunchKernelGGL((net_kernel<BS, IPT, XBAR, PP, DESC, 0>), dim3(groups / GROUPS), dim3(THREADS), 0,
                           stream, data);
    }
    else
    {
        hipLaunchKernelGGL((net_kernel<BS, IPT, XBAR, PP, DESC, 1>), dim3(groups / GROUPS), dim3(THREADS), 0,
                           stream, data);
    }
    return hipGetLastError() == hipSuccess ? 0 : 3;
}

template <int BS, int IPT, int XBAR, bool PP>
int by_order(int desc, int op, u64* data, int groups, hipStream_t stream)
{
    return desc != 0 ? launch<BS, IPT, XBAR, PP, true>(op, data, groups, stream)
                     : launch<BS, IPT, XBAR, PP, false>(op, data, groups, stream);
}

} // namespace

// Sorts (op 0) or merges (op 1) `groups` groups of bs*ipt keys in place.  Returns 0, 1 when the
// combination is not compiled, 2 for a group count that does not fill whole waves, 3 for a launch error.
extern "C" int nettest_run(int bs, int ipt, int xbar, int pp, int desc, int op, unsigned long long* data,
                           int groups, void* stream)
{
    auto* s = static_cast<hipStream_t>(stream);
    constexpr int X0 = bitsknn::XBAR_NONE;
    constexpr int X1 = bitsknn::XBAR_4_16_32;
#define CASE(BS, IPT, XB, PP)                                                                      \
    if (bs == BS && ipt == IPT && xbar == (XB) && (pp != 0) == PP)                                 \
    {                                                                                              \
        return by_order<BS, IPT, XB, PP>(desc, op, data, groups, s);                               \
    }
    // groups inside a wave (no LDS): the fused kernel's buffer sort (8 x 4) and list merges
    // (8 ... 64 lanes x 4 keys), the sampled radius of the top-k kernel (64 x 2, 4, 8)
    CASE(8, 4, X0, false)
    CASE(16, 4, X0, false)
    CASE(32, 4, X0, false)
    CASE(64, 4, X0, false)
    CASE(16, 2, X0, false)
    CASE(32, 1, X0, false)
    CASE(32, 2, X0, false)
    CASE(64, 1, X0, false)
    CASE(64, 2, X0, false)
    CASE(64, 8, X0, false)
    CASE(64, 4, X1, false)
    CASE(32, 4, X1, false)
    // whole workgroups: the top-k kernel's lists (crossbar exchanges, two LDS regions) and the
    // partial-bitonic kernel's (vector exchanges, one region); the reference's grid up to 1024 threads
    CASE(128, 1, X1, true)
    CASE(128, 2, X1, true)
    CASE(128, 16, X1, true)
    CASE(256, 1, X1, true)
    CASE(256, 8, X1, true)
    CASE(512, 1, X1, true)
    CASE(512, 4, X1, true)
    CASE(128, 1, X0, false)
    CASE(128, 4, X0, false)
    CASE(256, 2, X0, false)
    CASE(512, 4, X0, false)
    CASE(128, 8, X0, true)
    CASE(256, 4, X1, false)
    CASE(1024, 1, X0, false)
    CASE(1024, 2, X1, true)
#undef CASE
    return 1;
}
