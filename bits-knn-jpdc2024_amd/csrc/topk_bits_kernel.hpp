// bits top-k selection for gfx950 (wave64).
//
// One workgroup per matrix row.  The row is streamed from HBM in 16-byte loads; a value is kept
// only if its (value, label) key is below the current k-th smallest key ("radius").  Kept values
// are appended as 64-bit keys to a buffer in LDS.  When the buffer is full the whole workgroup
// sorts it descending with a bitonic network held in registers, takes the element-wise minimum
// with the ascending top-k list (a bitonic separator), re-sorts the resulting bitonic sequence
// and publishes the new radius.
//
// Same algorithm and phases as the reference kernel
// (include/bits/topk/singlepass/detail/bits_kernel.cuh:317-408: alloc :117-126, insert :277-302,
// merge :145-199, radius :30-51), laid out for 64-wide waves:
//  * every wave owns a private slice of the buffer, so appending needs no atomics: slots come
//    from a ballot-based prefix sum over the wave and a wave-uniform fill counter;
//  * the waves of a row do not synchronise per batch.  A wave whose slice is full raises a flag
//    in LDS and waits at a barrier; the others poll the flag once per batch and join.  The only
//    barriers are those of a merge;
//  * exchange distances below 64 lanes stay inside a wave, only distances of 64 lanes and more
//    go through LDS (two alternating regions, one barrier per exchange);
//  * the chunks of a row are visited both ends first and then front to back, so that sorted rows
//    of either direction tighten the radius at once, and for small batches the next chunk is
//    requested before the current one is filtered;
//  * long rows start from a radius taken from a sample of both row ends instead of from +inf,
//    which saves the first merges (they only halve the radius each);
//  * long lists also take an estimate of the k-th smallest value of the row from a sample spread
//    over the row, and repeat the row without it in the rare case that fewer than k values lie
//    below the estimate (a third of the values pass the filter then, and less than half the merges
//    are needed: 0.70 -> 0.79 of the HBM peak at k = 2048, 0.74-0.75 -> 0.83 at k = 512 with 128 and
//    256 threads per row).
// Because waves drift apart, the filter compares full keys when a value equals the radius, so
// that "equal values by lower label" holds no matter which wave saw which value first.

#ifndef BITSKNN_CSRC_TOPK_BITS_KERNEL_HPP_
#define BITSKNN_CSRC_TOPK_BITS_KERNEL_HPP_

#include "bitonic_net.hpp"
#include "common.hpp"

namespace bitsknn
{

typedef float vfloat4 __attribute__((ext_vector_type(4)));

struct topk_args
{
    const float* in;
    size_t in_stride;
    const std::int32_t* in_label;
    size_t label_stride;
    const std::int32_t* label_offsets;
    u32 cols;
    float* out_dist;
    std::int32_t* out_label;
    size_t out_stride;
    u32 k;
    // Rows cut into parts (the kernels instantiated with SQ only; parts <= 1 otherwise): rows
    // i*parts .. i*parts + parts - 1 of the matrix are the parts of logical row i.  out_dist and
    // out_label then take the k pairs of every part (row stride k), `done` holds one counter per
    // logical row (zero before the launch, zero again after it), and the workgroup that finishes
    // a logical row's last part selects the k smallest of its parts * k pairs, with their labels,
    // into final_dist / final_label.
    u32 parts;
    int* done;
    float* final_dist;
    std::int32_t* final_label;
    size_t final_stride;
};

// Merge the filled part of every wave's buffer slice into the ascending top-k list.  Slice w
// holds fill[w] keys from buffer[w*CAP].  The buffer memory doubles as exchange scratch once its
// keys are in registers.
template <int BS, int IPT>
__device__ __forceinline__ void merge_buffer(u64 (&topk)[IPT], u64* buffer, const int* fill, int t)
{
    constexpr int N = BS * IPT;
    constexpr int CAP = WAVE * IPT;
    u64 tmp[IPT];
#pragma unroll
    for (int r = 0; r < IPT; ++r)
    {
        const int idx = r * BS + t;
        tmp[r] = (idx % CAP) < fill[idx / CAP] ? buffer[idx] : PAD_KEY;
    }
    // LDS exchanges alternate between the N keys after the buffer and the buffer itself,
    // starting with the former: by the time the buffer is overwritten every thread has passed the
    // barrier of the first exchange and so has read its keys above.  One barrier per exchange.
    int flip = 1;
    net_sort<BS, IPT, 2, true, XBAR_4_16_32, true>(tmp, buffer, t, flip);
    // ascending list vs descending buffer: element-wise minimum keeps the N smallest of the 2N
    // keys and leaves them as a bitonic sequence
#pragma unroll
    for (int r = 0; r < IPT; ++r)
    {
        topk[r] = tmp[r] < topk[r] ? tmp[r] : topk[r];
    }
    net_phase<BS, IPT, N, N / 2, false, XBAR_4_16_32, true>(topk, buffer, t, flip);
}

// key of sorted element k-1, broadcast to the whole workgroup (includes a barrier)
template <int IPT>
__device__ __forceinline__ u64 broadcast_radius(const u64 (&topk)[IPT], u32 k, u64* slot, int t)
{
#pragma unroll
    for (int r = 0; r < IPT; ++r)
    {
        if (static_cast<u32>(t * IPT + r) == k - 1)
        {
            *slot = topk[r];
        }
    }
    __syncthreads();
    return *slot;
}

// Inserts `value` into the ascending array `lo` of the KEEP smallest values seen, dropping the
// largest (a NaN is taken for +inf).
template <int KEEP>
__device__ __forceinline__ void keep_smallest(float (&lo)[KEEP], float value)
{
    value = fminf(value, __builtin_inff());
#pragma unroll
    for (int j = KEEP - 1; j > 0; --j)
    {
        lo[j] = __builtin_amdgcn_fmed3f(value, lo[j - 1], lo[j]);
    }
    lo[0] = fminf(value, lo[0]);
}

// BS threads, IPT list entries per thread, L 16-byte (or 4 x 4-byte when !VEC) loads in flight
// per thread and iteration.  SQ: rows cut into parts (topk_args::parts): the workgroup that
// finishes the last part of a logical row goes through the kernel's body a second time, over the
// pairs its parts have left (reference: the second pass of single_query_bits,
// src/topk/singlepass/bits_knn.cu:132-186, there a launch of its own).
template <int BS, int IPT, int L, bool VEC, bool SQ = false>
__global__ void __launch_bounds__(BS) bits_topk_kernel(const topk_args a)
{
    constexpr int NL = BS * IPT;     // length of the top-k list and of the whole buffer
    constexpr int W = BS / WAVE;     // waves per row
    constexpr int CAP = WAVE * IPT;  // buffer slots owned by one wave (NL / W)
    constexpr int E = 4 * L;         // values per thread and iteration
    constexpr u32 CHUNK = BS * E;    // values per workgroup and iteration
    static_assert(E <= 32, "one pass bit per value in a 32-bit lane mask");
    // The sample that gives the first radius: smallest values kept per thread (the wave's pick
    // should not lie above the middle of what its lanes keep, and a wave picks up to 64 * IPT),
    // and 16-byte pieces per thread and end of the row (4 values looked at per value kept).
    constexpr int SAMPLE_KEEP = IPT <= 1 ? 2 : (IPT == 2 ? 4 : 8);
    constexpr u32 SAMPLE_PAIRS = SAMPLE_KEEP;
    // Lists of 1024 entries and more, and lists of 256 and more with at least two entries per
    // thread, also take an estimate of the k-th smallest value (see below): a sample of up to
    // EST_PIECES 16-byte pieces per thread, 2^14 values, spread over the row, of which every thread
    // keeps its EST_KEEP smallest.  (With one entry per thread -- 512 threads up to k = 512, 256
    // up to k = 256 -- the merges are cheap and the estimate costs more than it saves: 0.83 ->
    // 0.77-0.82 of the HBM peak at k = 512.)
    constexpr bool ESTIMATE = NL >= 1024 || (NL >= 256 && IPT >= 2);
    constexpr u32 EST_PIECES = 4096 / BS;
    constexpr int EST_KEEP = 8;

    __shared__ u64 buffer[2 * NL];   // candidates; the second half is exchange space of the merges
    __shared__ u64 s_radius;
    __shared__ int s_fill[W];
    __shared__ int s_flag;  // some wave wants a merge
    __shared__ int s_more;  // some wave still has values to process after this merge
    __shared__ u32 s_sample[W];
    __shared__ int s_ticket;

    int t = static_cast<int>(threadIdx.x);
    const int lane = t & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(t / WAVE);
    const size_t row_idx = blockIdx.x;
    // (with SQ the second turn of the loop below points these at the pairs of the row's parts)
    const float* row = a.in + row_idx * a.in_stride;
    const std::int32_t* lrow = a.in_label != nullptr ? a.in_label + row_idx * a.label_stride : nullptr;
    u32 label_offset = a.label_offsets != nullptr ? static_cast<u32>(a.label_offsets[row_idx]) : 0U;
    u32 n = a.cols;
    float* out_d = a.out_dist + row_idx * a.out_stride;
    std::int32_t* out_l = a.out_label + row_idx * a.out_stride;
    if constexpr (SQ)
    {
        // part p of a logical row: its labels start at p * (values per part)
        label_offset = static_cast<u32>(row_idx % a.parts) * a.cols;
    }
    u64* const slice = buffer + wave * CAP;
    for (int phase = 0; phase < (SQ ? 2 : 1); ++phase)
    {

    auto label_of = [&](u32 col) -> std::int32_t {
        const u32 base = lrow != nullptr ? static_cast<u32>(lrow[col]) : col;
        return static_cast<std::int32_t>(base + label_offset);
    };

    // column of value j of this thread within a chunk
    auto column_of = [&](u32 chunk, int j) -> u32 {
        if constexpr (VEC)
        {
            return chunk + static_cast<u32>(((j / 4) * BS + t) * 4 + (j % 4));
        }
        else
        {
            return chunk + static_cast<u32>(j * BS + t);
        }
    };

    u64 topk[IPT];

    // ---- radius from a sample.  Every thread looks at up to SAMPLE_PAIRS pairs of 16-byte pieces
    // of the row, one at its front and one at its back (at most a sixteenth of the row in all), and
    // keeps its SAMPLE_KEEP smallest values; every wave takes the c-th smallest of its
    // 64 * SAMPLE_KEEP, c = ceil(k / W).  At least k values of the row are then not above the
    // largest of these W values, so nothing above it can belong to the result: it serves as
    // radius until the list itself has a smaller one.  This replaces the first merges of a row,
    // which each only halve the radius and which all rows of a launch do at the same time.
    //
    // Lists of two and more entries per thread (ESTIMATE) on rows of at least 256 * BS values also
    // take an estimate, which counts where it lies below that bound (on uniform rows it does by far;
    // on sorted rows, whose ends hold the smallest values, the guaranteed bound is the lower one).
    // The sample is spread evenly over the row (at most a 64th of it) and the radius is its
    // value of rank e + 5 sqrt(e) + 2, where e = k * sample size / n values of the sample are
    // expected among the k smallest of the row: fewer than k values of the row lie below it with
    // a probability under 10^-5 per row when the sample is representative, whatever the order of
    // the row (sorted rows included).  At k = 2048 on rows of 2^20 uniform values 4 thousand values
    // pass the filter then instead of 12 thousand, and 3 merges are needed instead of 7.  The
    // estimate is not trusted: if the k-th key of the list has not got below it by the end of the
    // row, the pass is repeated from the guaranteed bound.
    bool estimated = false;
    u32 estimate = 0xFFFFFFFFU; // (the same in every wave)
    {
        u32 wave_bound = 0xFFFFFFFFU;
        if constexpr (ESTIMATE)
        {
            const u32 fit = n / (256U * BS);
            const u32 pieces = fit < EST_PIECES ? fit : EST_PIECES;
            const float expect =
                static_cast<float>(a.k) * static_cast<float>(pieces * 4 * BS) / static_cast<float>(n);
            const u32 rank = static_cast<u32>(ceilf(expect + 5.0F * sqrtf(expect))) + 2;
            if (pieces > 0 && a.k > 0 && rank <= WAVE)
            {
                const u32 segment = (n / pieces) & ~3U;
                const u32 offset = (segment / 2 - 2 * BS) & ~3U; // the piece sits in the middle
                float lo[EST_KEEP]; // ascending
#pragma unroll
                for (int j = 0; j < EST_KEEP; ++j)
                {
                    lo[j] = __builtin_inff();
                }
#pragma unroll 2
                for (u32 p = 0; p < pieces; ++p)
                {
                    const u32 col = p * segment + offset + static_cast<u32>(t) * 4;
                    vfloat4 x;
                    if constexpr (VEC)
                    {
                        x = *reinterpret_cast<const vfloat4*>(row + col);
                    }
                    else
                    {
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                        {
                            x[i] = row[col + i];
                        }
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                    {
                        keep_smallest(lo, x[i]);
                    }
                }
                u64 keys[EST_KEEP];
#pragma unroll
                for (int j = 0; j < EST_KEEP; ++j)
                {
                    keys[j] = static_cast<u64>(float_key(lo[j])) << 32U;
                }
                net_sort<WAVE, EST_KEEP, 2, false>(keys, nullptr, lane);
                // the 64 smallest of every wave (sorted position p is entry p % EST_KEEP of lane
                // p / EST_KEEP) meet in LDS; every wave sorts all of them and takes the same pick
                u32* const meet = reinterpret_cast<u32*>(buffer);
                if (lane < WAVE / EST_KEEP)
                {
#pragma unroll
                    for (int j = 0; j < EST_KEEP; ++j)
                    {
                        meet[wave * WAVE + lane * EST_KEEP + j] = static_cast<u32>(keys[j] >> 32U);
                    }
                }
                __syncthreads();
                u64 all[W];
#pragma unroll
                for (int i = 0; i < W; ++i)
                {
                    all[i] = static_cast<u64>(meet[i * WAVE + lane]) << 32U;
                }
                net_sort<WAVE, W, 2, false>(all, nullptr, lane);
                u32 pick = 0;
#pragma unroll
                for (int i = 0; i < W; ++i)
                {
                    pick = (rank - 1) % W == static_cast<u32>(i) ? static_cast<u32>(all[i] >> 32U) : pick;
                }
                estimate = static_cast<u32>(__builtin_amdgcn_readlane(
                    static_cast<int>(pick), static_cast<int>((rank - 1) / W)));
            }
        }
        // (the guaranteed bound is taken as well: on sorted rows, whose ends hold the smallest
        // values, it lies far below any estimate from a spread sample; the lower of the two counts)
        const u32 c = (a.k + W - 1) / W;
        const u32 fit = n / (128U * BS);
        // (next to an estimate one pair of pieces is enough: it is there for the sorted rows; lists
        // of 1024 entries and more do without it, where it costs 1-1.5 % on uniform rows)
        const u32 wanted = estimate != 0xFFFFFFFFU ? (NL >= 1024 ? 0U : 1U) : SAMPLE_PAIRS;
        const u32 pairs = fit < wanted ? fit : wanted;
        if (c <= WAVE * SAMPLE_KEEP && pairs > 0)
        {
            const u32 back = VEC ? (n - pairs * 4 * BS) & ~3U : n - pairs * 4 * BS;
            float lo[SAMPLE_KEEP]; // ascending
#pragma unroll
            for (int j = 0; j < SAMPLE_KEEP; ++j)
            {
                lo[j] = __builtin_inff();
            }
            for (u32 p = 0; p < pairs; ++p)
            {
                const u32 col = (p * BS + static_cast<u32>(t)) * 4;
                vfloat4 x[2];
                if constexpr (VEC)
                {
                    x[0] = *reinterpret_cast<const vfloat4*>(row + col);
                    x[1] = *reinterpret_cast<const vfloat4*>(row + back + col);
                }
                else
                {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                    {
                        x[0][i] = row[col + i];
                        x[1][i] = row[back + col + i];
                    }
                }
#pragma unroll
                for (int i = 0; i < 8; ++i)
                {
                    keep_smallest(lo, x[i / 4][i % 4]);
                }
            }
            u64 keys[SAMPLE_KEEP];
#pragma unroll
            for (int j = 0; j < SAMPLE_KEEP; ++j)
            {
                keys[j] = static_cast<u64>(float_key(lo[j])) << 32U;
            }
            net_sort<WAVE, SAMPLE_KEEP, 2, false>(keys, nullptr, lane);
            // sorted position c - 1 is entry (c - 1) % SAMPLE_KEEP of lane (c - 1) / SAMPLE_KEEP
            u32 pick = 0;
#pragma unroll
            for (int j = 0; j < SAMPLE_KEEP; ++j)
            {
                pick = (c - 1) % SAMPLE_KEEP == static_cast<u32>(j) ? static_cast<u32>(keys[j] >> 32U) : pick;
            }
            wave_bound = static_cast<u32>(__builtin_amdgcn_readlane(
                static_cast<int>(pick), static_cast<int>((c - 1) / SAMPLE_KEEP)));
        }
        s_sample[wave] = wave_bound;
    }

    // (a second turn of this loop only after an estimate that proved too low)
    for (bool again = false;; again = true)
    {
        if constexpr (ESTIMATE)
        {
            // (the thread index made opaque per turn: what is derived from it is then computed in
            // the turn rather than kept in registers around the whole loop, which costs 16 of them)
            asm volatile("" : "+v"(t));
        }
#pragma unroll
        for (int r = 0; r < IPT; ++r)
        {
            topk[r] = PAD_KEY;
        }
        if (t == 0)
        {
            s_flag = 0;
            s_more = 0;
        }
        __syncthreads();

        float radius = __builtin_inff();
        u64 radius_key = PAD_KEY;
        u64 first_key = PAD_KEY; // the radius the pass starts from
        bool sampled = false;
        {
            u32 bound = 0;
#pragma unroll
            for (int w = 0; w < W; ++w)
            {
                bound = s_sample[w] > bound ? s_sample[w] : bound;
            }
            // values up to the bound pass: the radius is the next key after it with the lowest label
            bound = static_cast<u32>(__builtin_amdgcn_readfirstlane(static_cast<int>(bound)));
            // (the estimate counts in the first turn only, and only where it is the lower one)
            estimated = !again && estimate < bound;
            bound = estimated ? estimate : bound;
            if (bound < float_key(__builtin_inff()))
            {
                radius_key = static_cast<u64>(bound + 1) << 32U;
                first_key = radius_key;
                radius = key_float(bound + 1);
                sampled = true;
            }
        }

        // Without a radius from the sample the first NL values go straight to the buffer and the
        // first merge sorts them; with one, they are filtered like the rest of the row (`head` = 0),
        // which saves that merge.
        const u32 head = sampled ? 0U : static_cast<u32>(NL);
        const u32 first = n < head ? n : head;
        const u32 full_end = n > head ? head + ((n - head) / CHUNK) * CHUNK : head;
        // The chunks after the head are visited in the order last, first, second, third, ...: both ends
        // of the row first, then front to back.  Whichever end of a sorted row holds the small values,
        // the radius is tight after the first NL values (ascending rows) or after the last chunk
        // (descending rows), where a plain front-to-back pass over a descending row would let every
        // value through the filter.  After the two ends the columns only grow, so a value that ties with
        // the radius soon has the larger label and fails the filter without a look at its key (rows of
        // few distinct values), and the loads walk through the row in address order.  The result does
        // not depend on the order.
        // (Measured against an order that alternates between the ends all the way in, on 1024 x 2^20
        // uniform values and on sorted and 256-valued rows of 65536: 0.1 % to 2 % of the HBM roofline
        // better in every case.)
        // (Lists of 512 entries and more visit the first chunk before the last -- first, last, second,
        // ... --: measured on uniform rows of 2^20 values they lose 0.4 % at k = 512 and 1.5 % at
        // k = 2048 of the HBM roofline with the back first, more than a merge per sorted row is worth
        // there.)
        const u32 chunk_count = n > head ? (n - head + CHUNK - 1) / CHUNK : 0;
        u32 left = chunk_count;            // chunks not yet visited
        constexpr bool BACK_FIRST = NL < 512;
        const std::int32_t span = chunk_count > 0 ? static_cast<std::int32_t>((chunk_count - 1) * CHUNK) : 0;
        // distance from the chunk being visited to the next one: to the other end, back to the second
        // chunk, then one chunk at a time
        std::int32_t jump = BACK_FIRST ? -span : span;
        u32 chunk = head + (BACK_FIRST ? static_cast<u32>(span) : 0U); // the next chunk to visit

        // the head goes straight to the buffer: column c into slot c (the barrier at the top of the
        // main loop orders these writes before the merge that reads them)
#pragma unroll
        for (int r = 0; r < IPT; ++r)
        {
            const u32 col = static_cast<u32>(r * BS + t);
            if (col < first)
            {
                buffer[col] = make_key(row[col], label_of(col));
            }
        }
        u32 cur_chunk = 0; // first column of the chunk held in v[]

        float v[E];
#pragma unroll
        for (int j = 0; j < E; ++j)
        {
            v[j] = 0.0F;
        }
        // the values of the chunk that starts at column `first`, value j of thread t as column_of says
        auto load_chunk = [&](float (&dst)[E], u32 first) {
            if (first < full_end)
            {
                if constexpr (VEC)
                {
                    const vfloat4* __restrict__ p = reinterpret_cast<const vfloat4*>(row + first) + t;
#pragma unroll
                    for (int l = 0; l < L; ++l)
                    {
                        const vfloat4 x = __builtin_nontemporal_load(p + l * BS);
                        dst[4 * l + 0] = x.x;
                        dst[4 * l + 1] = x.y;
                        dst[4 * l + 2] = x.z;
                        dst[4 * l + 3] = x.w;
                    }
                }
                else
                {
                    const float* __restrict__ p = row + first + t;
#pragma unroll
                    for (int j = 0; j < E; ++j)
                    {
                        dst[j] = __builtin_nontemporal_load(p + j * BS);
                    }
                }
            }
            else
            {
                // ragged tail: bounds-checked 4-byte loads in the same value-to-thread mapping
#pragma unroll
                for (int j = 0; j < E; ++j)
                {
                    const u32 col = column_of(first, j);
                    dst[j] = col < n ? row[col] : __builtin_inff();
                }
            }
        };
        // Software pipelining for small batches: the next chunk is requested before the current one
        // is filtered, at the price of E more registers and E moves per chunk.  Rows of two waves
        // (128 threads) leave 8 waves per compute unit, which need the depth also with 4 loads each.
        constexpr bool PIPE = L <= 2 || (BS == 128 && L <= 4);
        float ahead[E];
#pragma unroll
        for (int j = 0; j < E; ++j)
        {
            ahead[j] = 0.0F;
        }
        if constexpr (PIPE)
        {
            if (left > 0)
            {
                load_chunk(ahead, chunk);
            }
        }

        // Fill of this wave's slice (wave-uniform).  Passing values take slots in the order
        // (value index j, lane): value j of the lanes in its pass mask gets consecutive slots after
        // those of the values before it.
        //
        // Only when a chunk does not fit into the slice is per-lane state kept for it: bit j of
        // my_pass says value j of this lane passed the filter (decided with the radius of that
        // moment), slot_base is the slot of the chunk's first passing value.  A merge empties every
        // slice, so slot_base drops by CAP; a value is written in the round where its slot falls
        // into [0, CAP).
        int fill = static_cast<int>(first) - wave * CAP;
        fill = fill < 0 ? 0 : (fill > CAP ? CAP : fill);
        u32 my_pass = 0;
        int slot_base = 0;
        bool pending = false; // values of the chunk in v[] still wait for a slot

        auto lane_rank = [&](u64 mask) -> int {
            return static_cast<int>(__builtin_amdgcn_mbcnt_hi(
                static_cast<u32>(mask >> 32U), __builtin_amdgcn_mbcnt_lo(static_cast<u32>(mask), 0U)));
        };

        // exact filter: below the radius key (an equal value is decided by its label; the +inf
        // padding of a ragged tail never passes).  A NaN counts as +inf: it is neither below nor above
        // the radius and its key decides, which can only succeed while the radius is +inf.
        auto passes = [&](float value, int j) -> bool {
            bool pass = value < radius;
            if (!(value < radius) && !(value > radius))
            {
                const u32 col = column_of(cur_chunk, j);
                pass = col < n && make_key(value, label_of(col)) < radius_key;
            }
            return pass;
        };

        // writes the pending values whose slot is inside the slice; returns the end of the
        // chunk's reservation
        auto write_pending = [&]() -> int {
            int running = slot_base;
#pragma unroll
            for (int j = 0; j < E; ++j)
            {
                const bool mine = ((my_pass >> j) & 1U) != 0;
                const u64 mask = __builtin_amdgcn_ballot_w64(mine);
                if (mask != 0)
                {
                    const int slot = running + lane_rank(mask);
                    if (mine && slot >= 0 && slot < CAP)
                    {
                        const u32 col = column_of(cur_chunk, j);
                        slice[slot] = make_key(v[j], label_of(col));
                    }
                    running += __popcll(mask);
                }
            }
            return running;
        };

        for (;;)
        {
            // ---- rendezvous: every wave arrives here when it needs a merge, saw the flag, or ran
            // out of values
            const bool more_work = pending || left > 0;
            // (wave-uniform values, stored by every lane: a branch on the lane next to a loop exit
            // makes the compiler treat the loop state as differing between lanes, which turns the
            // streaming loop into an exec-masked one with its counters in vector registers)
            s_fill[wave] = fill;
            if (more_work)
            {
                s_more = 1;
            }
            __syncthreads();
            // (the same in every lane; said explicitly so that the loops stay wave-uniform)
            int total = 0;
#pragma unroll
            for (int w = 0; w < W; ++w)
            {
                total += s_fill[w];
            }
            total = __builtin_amdgcn_readfirstlane(total);
            const bool more = __builtin_amdgcn_readfirstlane(s_more) != 0;
            if (total > 0)
            {
                merge_buffer<BS, IPT>(topk, buffer, s_fill, t);
                // the barriers of the merge lie between the reads above and this reset; the barrier
                // of the broadcast publishes it together with the radius
                if (t == 0)
                {
                    s_flag = 0;
                    s_more = 0;
                }
                // (the radius from the sample stays until the list has a smaller one)
                const u64 list_radius = broadcast_radius<IPT>(topk, a.k, &s_radius, t);
                radius_key = list_radius < radius_key ? list_radius : radius_key;
                radius = key_value(radius_key);
            }
            else
            {
                __syncthreads(); // orders the reads above before the reset below
                if (t == 0)
                {
                    s_flag = 0;
                    s_more = 0;
                }
                __syncthreads();
            }
            if (!more)
            {
                break;
            }
            fill = 0;
            if (pending)
            {
                slot_base -= CAP;
                const int end = write_pending();
                if (end > CAP)
                {
                    fill = CAP;
                    s_flag = 1;
                    continue;
                }
                fill = end;
                pending = false;
            }

            // ---- streaming: no synchronisation with the other waves except polling the flag
            while (left > 0)
            {
                if constexpr (PIPE)
                {
                    // the values of this chunk were requested an iteration (or a merge) ago
#pragma unroll
                    for (int j = 0; j < E; ++j)
                    {
                        v[j] = ahead[j];
                    }
                }
                else
                {
                    load_chunk(v, chunk);
                }
                const int flag = __hip_atomic_load(&s_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                cur_chunk = chunk;
                left -= 1;
                chunk += static_cast<u32>(jump);
                jump = left + 1 == chunk_count && !BACK_FIRST ? static_cast<std::int32_t>(CHUNK) - span
                                                              : static_cast<std::int32_t>(CHUNK);
                if constexpr (PIPE)
                {
                    // request the next chunk before this one is filtered: the loads stay in flight
                    // through the filter and through a merge, if one comes
                    if (left > 0)
                    {
                        load_chunk(ahead, chunk);
                    }
                }

                // NaN-propagating minimum (v_minimum3_f32): a lane that holds a NaN of any kind gets a NaN
                // here and takes the look at every value below (the NaN-ignoring minimum would need
                // every operand quietened first, and loses values after a signalling NaN otherwise)
                float smallest = v[0];
#pragma unroll
                for (int j = 1; j < E; ++j)
                {
                    smallest = __builtin_elementwise_minimum(smallest, v[j]);
                }
                // A value equal to the radius passes only with a label below the radius key's.  With
                // implicit labels every label of this chunk is at least that of its first column, so
                // when that one is not below, equal values need no look (rows with few distinct
                // values have one in every chunk).
                const bool no_ties =
                    lrow == nullptr && static_cast<std::int32_t>(cur_chunk + label_offset) >= key_label(radius_key);
                // (negated compares: true for a NaN)
                if (__builtin_amdgcn_ballot_w64(no_ties ? !(smallest >= radius) : !(smallest > radius)) != 0)
                {
                    int running = fill;
#pragma unroll
                    for (int j = 0; j < E; ++j)
                    {
                        if (__builtin_amdgcn_ballot_w64(!(v[j] > radius)) != 0)
                        {
                            const bool pass = passes(v[j], j);
                            const u64 mask = __builtin_amdgcn_ballot_w64(pass);
                            if (mask != 0)
                            {
                                const int slot = running + lane_rank(mask);
                                if (pass && slot < CAP)
                                {
                                    const u32 col = column_of(cur_chunk, j);
                                    slice[slot] = make_key(v[j], label_of(col));
                                }
                                running += __popcll(mask);
                            }
                        }
                    }
                    if (running > CAP)
                    {
                        // the slice is full: remember which values passed (the radius changes with
                        // the merge) and ask for a merge
                        my_pass = 0;
#pragma unroll
                        for (int j = 0; j < E; ++j)
                        {
                            my_pass |= passes(v[j], j) ? (1U << j) : 0U;
                        }
                        slot_base = fill;
                        pending = true;
                        fill = CAP;
                        s_flag = 1;
                        break;
                    }
                    fill = running;
                }
                if (__builtin_amdgcn_readfirstlane(flag) != 0)
                {
                    break;
                }
            }
        }

        if constexpr (ESTIMATE)
        {
            // Everything the filter dropped was not below the radius of that moment, and no radius
            // was above the first one.  If the k-th key of the list got below the first radius, the
            // dropped values all lie above the list; if not, fewer than k values of the row lie
            // below the estimate, and the row is done again without it.
            const u32 high = static_cast<u32>(__builtin_amdgcn_readfirstlane(static_cast<int>(radius_key >> 32U)));
            const u32 low = static_cast<u32>(__builtin_amdgcn_readfirstlane(static_cast<int>(radius_key)));
            if (estimated && !(((static_cast<u64>(high) << 32U) | low) < first_key))
            {
                estimated = false;
                continue;
            }
        }
        break;
    }

    // (the pairs of a part are stored past the caches of this part of the chip, so that the workgroup
    // that reduces the row, wherever it runs, finds them without a write-back of the whole cache)
    const bool to_be_reduced = SQ && phase == 0 && a.parts > 1 && a.done != nullptr;
#pragma unroll
    for (int r = 0; r < IPT; ++r)
    {
        const u32 e = static_cast<u32>(t * IPT + r);
        if (e < a.k)
        {
            if (to_be_reduced)
            {
                __hip_atomic_store(out_d + e, key_value(topk[r]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(out_l + e, key_label(topk[r]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            else
            {
                out_d[e] = key_value(topk[r]);
                out_l[e] = key_label(topk[r]);
            }
        }
    }
    if constexpr (SQ)
    {
        if (!to_be_reduced)
        {
            break;
        }
        // The barrier waits for the stores of every thread; then one thread counts the part in.
        // The workgroup that counts in last sees the pairs of all parts of its logical row (it
        // drops what its caches hold first) and selects from them.
        __syncthreads();
        const size_t logical = row_idx / a.parts;
        if (t == 0)
        {
            s_ticket = __hip_atomic_fetch_add(a.done + logical, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
        if (s_ticket != static_cast<int>(a.parts) - 1)
        {
            break;
        }
        if (t == 0)
        {
            a.done[logical] = 0; // for the next launch
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        const size_t first_part = logical * a.parts;
        row = a.out_dist + first_part * a.out_stride;
        lrow = a.out_label + first_part * a.out_stride;
        label_offset = 0;
        n = a.parts * a.k;
        out_d = a.final_dist + logical * a.final_stride;
        out_l = a.final_label + logical * a.final_stride;
        __syncthreads();
    }
    } // phase
}


} // namespace bitsknn

#endif // BITSKNN_CSRC_TOPK_BITS_KERNEL_HPP_
