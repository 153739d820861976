// Test-only timing probes of how gfx950 issues fp32 matrix instructions next to vector instructions:
// the measurements the fused and distance kernels were shaped by (loaded by
// tests/test_y_issue_probe_gpu.py, built into tests/libissueprobe.so).  Nothing in the library uses
// this file.
//
//  * chain:   nothing but v_mfma_f32_32x32x2_f32, CHAINS independent accumulator chains per wave;
//  * fma:     two chains, and after every matrix instruction V vector multiply-adds on registers
//             of their own (no dependence on the matrix results): do they overlap with it?
//  * filter:  per iteration a pair of 32 x 32 tiles of STEPS matrix instructions each, then the fused
//             kernel's filter over both (a compare, a tree of seven v_min3, a compare, one branch).
//
// Every workgroup has 4 waves (one per SIMD); `workgroups_per_cu` of them share a compute unit.

#include <hip/hip_runtime.h>

#include <cstdint>

namespace
{

typedef float vfloat16 __attribute__((ext_vector_type(16)));
using u64 = unsigned long long;

__device__ __forceinline__ float min3(float a, float b, float c)
{
    float r;
    asm("v_min3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

template <int CHAINS>
__global__ void __launch_bounds__(256) chain_kernel(float* out, int iters, float av, float bv)
{
    vfloat16 acc[CHAINS];
#pragma unroll
    for (int c = 0; c < CHAINS; ++c)
    {
#pragma unroll
        for (int r = 0; r < 16; ++r)
        {
            acc[c][r] = 0.0F;
        }
    }
    const float a = av + static_cast<float>(threadIdx.x);
    for (int i = 0; i < iters; ++i)
    {
#pragma unroll
        for (int c = 0; c < CHAINS; ++c)
        {
            acc[c] = __builtin_amdgcn_mfma_f32_32x32x2f32(a + static_cast<float>(c), bv, acc[c], 0, 0, 0);
        }
    }
    float s = 0.0F;
#pragma unroll
    for (int c = 0; c < CHAINS; ++c)
    {
#pragma unroll
        for (int r = 0; r < 16; ++r)
        {
            s += acc[c][r];
        }
    }
    if (s == 12345.678F)
    {
        out[threadIdx.x] = s;
    }
}

template <int V>
__global__ void __launch_bounds__(256) fma_kernel(float* out, int iters, float av, float bv)
{
    vfloat16 acc0;
    vfloat16 acc1;
#pragma unroll
    for (int r = 0; r < 16; ++r)
    {
        acc0[r] = 0.0F;
        acc1[r] = 0.0F;
    }
    float x[V > 0 ? V : 1];
#pragma unroll
    for (int v = 0; v < (V > 0 ? V : 1); ++v)
    {
        x[v] = av * static_cast<float>(v + 1);
    }
    const float a = av + static_cast<float>(threadIdx.x);
    for (int i = 0; i < iters; ++i)
    {
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, bv, acc0, 0, 0, 0);
#pragma unroll
        for (int v = 0; v < V; ++v)
        {
            asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x[v]) : "v"(bv), "v"(av));
        }
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a + 1.0F, bv, acc1, 0, 0, 0);
#pragma unroll
        for (int v = 0; v < V; ++v)
        {
            asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x[v]) : "v"(bv), "v"(av));
        }
    }
    float s = 0.0F;
#pragma unroll
    for (int r = 0; r < 16; ++r)
    {
        s += acc0[r] + acc1[r];
    }
#pragma unroll
    for (int v = 0; v < (V > 0 ? V : 1); ++v)
    {
        s += x[v];
    }
    if (s == 12345.678F)
    {
        out[threadIdx.x] = s;
    }
}

// the fused kernel's test of one tile: true if any of the lane's 16 values lies below `radius`
__device__ __forceinline__ bool tile_passes(const vfloat16& acc, float radius)
{
    const u64 last = __builtin_amdgcn_ballot_w64(acc[15] < radius);
    __builtin_amdgcn_sched_barrier(0);
    float low[5];
#pragma unroll
    for (int g = 0; g < 5; ++g)
    {
        low[g] = min3(acc[3 * g], acc[3 * g + 1], acc[3 * g + 2]);
    }
    const float smallest = min3(min3(low[0], low[1], low[2]), low[3], low[4]);
    return (last | __builtin_amdgcn_ballot_w64(smallest < radius)) != 0;
}

template <int STEPS, bool FILTER>
__global__ void __launch_bounds__(256) filter_kernel(float* out, int iters, float av, float bv, float radius)
{
    vfloat16 zero;
#pragma unroll
    for (int r = 0; r < 16; ++r)
    {
        zero[r] = av * static_cast<float>(r);
    }
    float a0 = av + static_cast<float>(threadIdx.x);
    float a1 = a0 * 0.37F;
    int hits = 0;
    for (int i = 0; i < iters; ++i)
    {
        vfloat16 acc0 = zero;
        vfloat16 acc1 = zero;
#pragma unroll
        for (int s = 0; s < STEPS; ++s)
        {
            acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, bv, acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, bv, acc1, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (FILTER)
        {
            if (tile_passes(acc0, radius))
            {
                hits += 1;
                out[hits] = acc0[3];
            }
            if (tile_passes(acc1, radius))
            {
                hits += 1;
                out[hits] = acc1[3];
            }
        }
        else
        {
            // one compare that needs both results, so that the pairs are not merged into one chain
            if (__builtin_amdgcn_ballot_w64(acc0[15] + acc1[15] < radius) != 0)
            {
                hits += 1;
                out[hits] = acc0[3];
            }
        }
        a0 += 1.0F;
        a1 += 0.7F;
    }
    if (hits == 12345)
    {
        out[threadIdx.x] = a0;
    }
}

template <typename Launch>
int timed(Launch launch, int iters, double* ms, hipStream_t stream)
{
    hipEvent_t start = nullptr;
    hipEvent_t stop = nullptr;
    if (hipEventCreate(&start) != hipSuccess || hipEventCreate(&stop) != hipSuccess)
    {
        return 1;
    }
    launch(16);
    int status = hipStreamSynchronize(stream) == hipSuccess ? 0 : 2;
    if (status == 0)
    {
        (void)hipEventRecord(start, stream);
        launch(iters);
        (void)hipEventRecord(stop, stream);
        status = hipEventSynchronize(stop) == hipSuccess && hipGetLastError() == hipSuccess ? 0 : 3;
    }
    float elapsed = 0.0F;
    if (status == 0 && hipEventElapsedTime(&elapsed, start, stop) != hipSuccess)
    {
        status = 4;
    }
    *ms = elapsed;
    (void)hipEventDestroy(start);
    (void)hipEventDestroy(stop);
    return status;
}

} // namespace

// kind 0: chain (param = chains: 1, 2, 4), kind 1: fma (param = vector instructions per matrix
// instruction: 0, 2, 4, 8), kind 2: matrix pairs without the filter, kind 3: with it (param = matrix
// instructions per tile: 4, 8, 16).  `scratch` holds at least 2^20 bytes of device memory.  Returns 0
// and the kernel time in *ms, -1 for an unknown combination, > 0 for a runtime error.
extern "C" int issue_probe_run(int kind, int param, int workgroups_per_cu, int compute_units, int iters,
                               float* scratch, double* ms, void* stream_ptr)
{
    hipStream_t stream = static_cast<hipStream_t>(stream_ptr);
    const dim3 grid(static_cast<unsigned>(workgroups_per_cu * compute_units));
    const dim3 block(256);
    if (workgroups_per_cu < 1 || workgroups_per_cu > 4 || compute_units < 1 || iters < 1 || scratch == nullptr ||
        ms == nullptr)
    {
        return -1;
    }
#define CHAIN_CASE(C)                                                                                        \
    if (kind == 0 && param == (C))                                                                           \
    {                                                                                                        \
        return timed([&](int n) { chain_kernel<C><<<grid, block, 0, stream>>>(scratch, n, 1.0F, 2.0F); },    \
                     iters, ms, stream);                                                                     \
    }
#define FMA_CASE(V)                                                                                          \
    if (kind == 1 && param == (V))                                                                           \
    {                                                                                                        \
        return timed([&](int n) { fma_kernel<V><<<grid, block, 0, stream>>>(scratch, n, 1.0F, 2.0F); },      \
                     iters, ms, stream);                                                                     \
    }
#define FILTER_CASE(S)                                                                                       \
    if (kind == 2 && param == (S))                                                                           \
    {                                                                                                        \
        return timed([&](int n) {                                                                            \
            filter_kernel<S, false><<<grid, block, 0, stream>>>(scratch, n, 1.0F, 2.0F, -1.0e30F);           \
        }, iters, ms, stream);                                                                               \
    }                                                                                                        \
    if (kind == 3 && param == (S))                                                                           \
    {                                                                                                        \
        return timed([&](int n) {                                                                            \
            filter_kernel<S, true><<<grid, block, 0, stream>>>(scratch, n, 1.0F, 2.0F, -1.0e30F);            \
        }, iters, ms, stream);                                                                               \
    }
    CHAIN_CASE(1)
    CHAIN_CASE(2)
    CHAIN_CASE(4)
    FMA_CASE(0)
    FMA_CASE(2)
    FMA_CASE(4)
    FMA_CASE(8)
    FILTER_CASE(4)
    FILTER_CASE(8)
    FILTER_CASE(16)
#undef CHAIN_CASE
#undef FMA_CASE
#undef FILTER_CASE
    return -1;
}
