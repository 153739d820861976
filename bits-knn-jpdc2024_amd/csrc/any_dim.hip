// bits-fused for vectors of more than 256 dimensions, where no stage of the matrix kernels fits into
// LDS any more: a plain kernel on the vector unit, one query per thread.  The reference's kernel
// takes any dimension from its lower bound on (src/topk/singlepass/fused_cache_knn.cu:63-67); this
// one is what keeps that true here.  It is not tuned: the dimensions the reference measures stop
// at 64.
//
// Arithmetic: the reference's -- norm and dot product by sequential fused multiply-adds over the
// dimensions in order, then norm - 2 dot (include/bits/topk/singlepass/
// fused_cache_kernel_structs.cuh:457-522, :622-631) -- so the lists equal the reference
// arithmetic's bit for bit, equal distances by lower index.
//
// A workgroup of 256 threads has 256 queries and walks through its range of points (blockIdx.y, as
// in the matrix kernels) in tiles of 16 points, 32 dimensions at a time: the tile's values go
// through LDS, where every thread reads them as broadcasts, its own query's 32 values come from
// global memory into registers.  The list of a query lives in the caller's output arrays
// (fused_args::out_dist / out_label, k entries): unordered while the points are visited, with its
// AD_TOP largest entries (keys, labels, positions) kept in registers.  A point that is nearer than
// the largest one replaces it and either joins those registers or leaves one entry fewer in them;
// only when they are used up is the list scanned again.  Its thread sorts the list at the end.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "common.hpp"
#include "fused_args.hpp"

namespace bitsknn
{

namespace
{

constexpr int AD_THREADS = 256; // queries per workgroup
constexpr int AD_POINTS = 16;   // points per tile
constexpr int AD_DIMS = 32;     // dimensions per step
constexpr int AD_TOP = 8;       // largest entries of a list that its thread keeps track of
constexpr std::int32_t AD_NO_LABEL = 0x7FFFFFFF;

typedef float vfloat4 __attribute__((ext_vector_type(4)));

// the order of the lists: a NaN counts as +inf (and is reported as it is)
__device__ __forceinline__ float order_key(float value)
{
    return value != value ? __builtin_inff() : value;
}

__global__ void __launch_bounds__(AD_THREADS) fused_any_dim_kernel(const fused_args a, const int k)
{
    __shared__ __align__(16) float tile[AD_POINTS][AD_DIMS];
    const int t = static_cast<int>(threadIdx.x);
    const int my_q = static_cast<int>(blockIdx.x) * AD_THREADS + t;
    const bool live = my_q < a.q;
    const float* const mine = a.queries + (live ? my_q : 0);
    const size_t total_points = static_cast<size_t>(a.n);
    const int n_begin = static_cast<int>(blockIdx.y) * a.split_points;
    const int n_end = a.n < n_begin + a.split_points ? a.n : n_begin + a.split_points;
    const size_t list_at = (static_cast<size_t>(live ? my_q : 0) * static_cast<size_t>(a.splits) + blockIdx.y) *
                           static_cast<size_t>(a.list_stride);
    float* const list_d = a.out_dist + list_at;
    std::int32_t* const list_l = a.out_label + list_at;
    if (live)
    {
        for (int i = 0; i < k; ++i)
        {
            list_d[i] = __builtin_inff();
            list_l[i] = AD_NO_LABEL;
        }
    }
    int fill = 0;                    // entries of the list that hold a point
    // the `tracked` largest entries of the full list, largest first (by key, then label); the
    // others are not above the last of them
    float top_key[AD_TOP];
    std::int32_t top_label[AD_TOP];
    int top_at[AD_TOP];
    int tracked = 0;
#pragma unroll
    for (int j = 0; j < AD_TOP; ++j)
    {
        top_key[j] = -__builtin_inff();
        top_label[j] = -1;
        top_at[j] = 0;
    }
    // (key, label) of an entry above that of another
    auto above = [](float key, std::int32_t label, float other, std::int32_t other_label) -> bool {
        return key > other || (key == other && label > other_label);
    };
    // puts an entry into the tracked ones where it belongs (the last one falls out if all are in use)
    auto track = [&](float key, std::int32_t label, int at) {
#pragma unroll
        for (int j = 0; j < AD_TOP; ++j)
        {
            const bool here = j < tracked ? above(key, label, top_key[j], top_label[j]) : true;
            if (here)
            {
                const float was_key = top_key[j];
                const std::int32_t was_label = top_label[j];
                const int was_at = top_at[j];
                top_key[j] = key;
                top_label[j] = label;
                top_at[j] = at;
                key = was_key;
                label = was_label;
                at = was_at;
            }
        }
    };
    // the staging of a tile: thread t carries point t % 16 in dimensions t / 16 and t / 16 + 16 of a step
    const int sp = t % AD_POINTS;
    const int sc = t / AD_POINTS;
    for (int p0 = n_begin; p0 < n_end; p0 += AD_POINTS)
    {
        float norm[AD_POINTS];
        float dot[AD_POINTS];
#pragma unroll
        for (int p = 0; p < AD_POINTS; ++p)
        {
            norm[p] = 0.0F;
            dot[p] = 0.0F;
        }
#pragma unroll 1
        for (int d0 = 0; d0 < a.dim; d0 += AD_DIMS)
        {
            float y[AD_DIMS];
#pragma unroll
            for (int c = 0; c < AD_DIMS; ++c)
            {
                // (a row that exists; dimensions from dim on count as zero on both sides)
                const int dd = d0 + c < a.dim ? d0 + c : 0;
                y[c] = mine[static_cast<size_t>(dd) * static_cast<size_t>(a.q)];
            }
            __syncthreads(); // the values of the step before have been read
#pragma unroll
            for (int h = 0; h < 2; ++h)
            {
                const int dd = d0 + sc + 16 * h;
                const int point = p0 + sp;
                float value = 0.0F;
                if (dd < a.dim && point < n_end)
                {
                    value = a.points[static_cast<size_t>(dd) * total_points + static_cast<size_t>(point)];
                }
                tile[sp][sc + 16 * h] = value;
            }
            __syncthreads();
#pragma unroll
            for (int p = 0; p < AD_POINTS; ++p)
            {
#pragma unroll
                for (int c = 0; c < AD_DIMS; c += 4)
                {
                    const vfloat4 x = *reinterpret_cast<const vfloat4*>(&tile[p][c]);
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                    {
                        const float u = d0 + c + i < a.dim ? y[c + i] : 0.0F;
                        norm[p] = __builtin_fmaf(x[i], x[i], norm[p]);
                        dot[p] = __builtin_fmaf(u, x[i], dot[p]);
                    }
                }
            }
        }
#pragma unroll 1
        for (int p = 0; p < AD_POINTS; ++p)
        {
            const float value = __builtin_fmaf(-2.0F, dot[p], norm[p]);
            const int label = p0 + p;
            const float key = order_key(value);
            if (!live || label >= n_end)
            {
                continue;
            }
            if (fill < k)
            {
                list_d[fill] = value;
                list_l[fill] = label;
                ++fill;
                if (fill < k)
                {
                    continue;
                }
            }
            else if (key < top_key[0])
            {
                // (labels come in ascending order: of equal distances the earlier point stays)
                const int at = top_at[0];
                list_d[at] = value;
                list_l[at] = label;
                // the largest entry is gone: the others move up
#pragma unroll
                for (int j = 0; j + 1 < AD_TOP; ++j)
                {
                    top_key[j] = top_key[j + 1];
                    top_label[j] = top_label[j + 1];
                    top_at[j] = top_at[j + 1];
                }
                --tracked;
                // the new entry is one of the tracked ones if it is above the last of them (everything
                // that is not tracked is not above that one)
                if (tracked > 0)
                {
                    bool joins = false;
#pragma unroll
                    for (int j = 0; j < AD_TOP; ++j)
                    {
                        joins = joins || (j == tracked - 1 && above(key, label, top_key[j], top_label[j]));
                    }
                    if (joins)
                    {
                        track(key, label, at);
                        ++tracked;
                    }
                    continue;
                }
            }
            else
            {
                continue;
            }
            // the list is full and nothing is tracked: its AD_TOP largest entries (all of a shorter list)
            tracked = 0;
            for (int i = 0; i < k; ++i)
            {
                const float there = order_key(list_d[i]);
                const std::int32_t its_label = list_l[i];
                bool in = tracked < AD_TOP;
#pragma unroll
                for (int jj = 0; jj < AD_TOP; ++jj)
                {
                    in = in || (jj == AD_TOP - 1 && above(there, its_label, top_key[jj], top_label[jj]));
                }
                if (in)
                {
                    track(there, its_label, i);
                    tracked = tracked < AD_TOP ? tracked + 1 : AD_TOP;
                }
            }
        }
    }
    // ascending by (distance, label); the entries from `fill` on hold no point and stay where they are
    if (live)
    {
        for (int i = 1; i < fill; ++i)
        {
            const float value = list_d[i];
            const std::int32_t label = list_l[i];
            const float key = order_key(value);
            int j = i;
            while (j > 0)
            {
                const float before = order_key(list_d[j - 1]);
                const std::int32_t label_before = list_l[j - 1];
                if (!(before > key || (before == key && label_before > label)))
                {
                    break;
                }
                list_d[j] = list_d[j - 1];
                list_l[j] = label_before;
                --j;
            }
            list_d[j] = value;
            list_l[j] = label;
        }
    }
}

} // namespace

hipError_t launch_fused_any_dim(const fused_args& a, int k, hipStream_t stream)
{
    const unsigned grid = static_cast<unsigned>((static_cast<long long>(a.q) + AD_THREADS - 1) / AD_THREADS);
    hipLaunchKernelGGL(fused_any_dim_kernel, dim3(grid, static_cast<unsigned>(a.splits)), dim3(AD_THREADS), 0, stream, a,
                       k);
    return hipGetLastError();
}

} // namespace bitsknn
