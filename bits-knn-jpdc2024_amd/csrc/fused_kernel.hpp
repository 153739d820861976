// bits-fused for gfx950: partial squared L2 distance (||p||^2 - 2 q.p) and top-k in one kernel.
// The q x n distance matrix never leaves the registers of the wave that computes it.
//
// Replaces the reference's fused_cache_kernel
// (include/bits/topk/singlepass/fused_cache_kernel_structs.cuh:663-800: distance tiles :315-632,
// per-query buffers and merges :25-305).  Same phases -- distance tile, filter against the k-th
// distance of each query, append to a per-query buffer, merge buffers into sorted top-k lists --
// laid out for the matrix cores and 64-wide waves:
//
//  * A workgroup of 4 waves owns 128 queries (32 per wave) and walks over its range of points in
//    stages of PT points, two stages in LDS (one being multiplied, one being filled; one barrier
//    per stage) or, for lists of up to 128 entries in up to 8 dimensions and of up to 32 entries in
//    16 to 128 dimensions or with bf16 pieces, a ring of three stages without barriers.
//    A stage is the MFMA A operand: rows 0..d-1 hold the points, the following rows
//    hold the staging threads' shares of ||p||^2, so that v_mfma_f32_32x32x2_f32 against the query
//    fragment (-2q_0..-2q_{d-1}, 1, 1) yields ||p||^2 - 2 q.p directly, the dot product accumulated
//    first and the norm added last.  For d <= 64 the norm is one row and the initial accumulator
//    instead.
//  * The query fragment stays in registers for the whole kernel.  In the 32 x 32 result tile a
//    lane holds 16 distances of ONE query (column), so the filter is a min-tree over 16
//    registers and one compare against that query's radius.
//  * Every query has a 32-slot buffer in LDS (64 slots for lists of 128 and more in up to 16
//    dimensions when the points are cut into ranges).  Slots are handed out without atomics: the two
//    lanes that share a query exchange their pass counts, and the fill is kept in a register.
//    Before a tile would overflow any buffer of the wave, the wave merges all its buffers; the
//    other waves of the workgroup, which would wait for it at the stage barrier, then merge
//    theirs in the same stage.
//  * The sorted top-k lists live in the output arrays themselves between merges, read back by the
//    lanes that wrote them (plain loads and stores, requested one pass ahead).  A merge is a
//    segmented bitonic network in registers, 4 keys per lane: 8 queries per pass for k <= 32;
//    for longer lists the buffers are sorted in place first (8 queries per pass) and then merged
//    into the lists of 4, 2 or 1 queries per pass.
//  * With few queries the points are cut into ranges (blockIdx.y) whose partial lists go to a
//    caller-provided workspace and are reduced by one bits top-k pass with explicit labels.
//
// Equal distances are ordered by lower point index: points are visited in index order, so a
// value equal to a query's radius can never displace what is already merged.

#ifndef BITSKNN_CSRC_FUSED_KERNEL_HPP_
#define BITSKNN_CSRC_FUSED_KERNEL_HPP_

#include <type_traits>

#include "bf16x3.hpp"
#include "bitonic_net.hpp"
#include "common.hpp"
#include "fused_args.hpp"

namespace bitsknn
{

namespace
{

// Instrumented build (-DBITSKNN_FUSED_TIMING): every wave adds up the cycles it spends in the phases
// of the stage loop of the ring (0 waiting for a stage, 1 waiting for the loads of the next one,
// 2 writing it and requesting the one after, 3 filtering the stage, 4 working through candidates)
// and adds them to fused_args::timing at the end.
#ifdef BITSKNN_FUSED_TIMING
#define BITSKNN_FT_LAP(i)                                                                          \
    do                                                                                            \
    {                                                                                             \
        const long long ft_now = static_cast<long long>(__builtin_readcyclecounter());            \
        ft_cycles[i] += ft_now - ft_mark;                                                         \
        ft_mark = ft_now;                                                                         \
    } while (0)
#else
#define BITSKNN_FT_LAP(i)                                                                          \
    do                                                                                            \
    {                                                                                             \
    } while (0)
#endif

// minimum of three values in one instruction; a NaN operand is ignored
__device__ __forceinline__ float min3(float a, float b, float c)
{
    float r;
    asm("v_min3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// the same, but a NaN operand gives a NaN
__device__ __forceinline__ float minimum3(float a, float b, float c)
{
    float r;
    asm("v_minimum3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

typedef __bf16 vbf16x2 __attribute__((ext_vector_type(2)));
typedef float vfloat2 __attribute__((ext_vector_type(2)));

// x[i] ~ x1 + x2 with two bf16 pieces rounded to nearest: x1 = bf16(x), x2 = bf16(x - x1) (the
// difference is exact), so |x - x1 - x2| <= 2^-16 |x|.  Piece c of values 2j and 2j+1 shares word j
// of pc (the layout of a matrix operand of 8 bf16 values).
__device__ __forceinline__ void cut_bf16x2(const float (&x)[8], vuint4& p1, vuint4& p2)
{
#pragma unroll
    for (int j = 0; j < 4; ++j)
    {
        const vfloat2 pair{x[2 * j], x[2 * j + 1]};
        const u32 first = __builtin_bit_cast(u32, __builtin_convertvector(pair, vbf16x2));
        const vfloat2 rest{pair.x - __builtin_bit_cast(float, first << 16U),
                           pair.y - __builtin_bit_cast(float, first & 0xFFFF0000U)};
        p1[j] = first;
        p2[j] = __builtin_bit_cast(u32, __builtin_convertvector(rest, vbf16x2));
    }
}

// Error budget of the filter of FUSED_ARITH_EXACT.  For a query q and a point p let
// V = fl(norm - 2 dot) be the reported value (sequential fused multiply-adds over the dimensions in
// order) and W the filter's value: the sum, on the bf16 matrix instructions with fp32 accumulation,
// of the lowered norm's two pieces and of the products of the pieces of -2q and p with the
// second-order terms left out.  With Q = ||q||^2, N = ||p||^2, S = N + 2 sum |q_i p_i| <= 2 N + Q:
//   |V - exact|          <= (d + 2) 2^-24 S                      (d <= 64: 4.0e-6 S)
//   pieces left out      <= 3 * 2^-16 (1 + 2^-7) * 2 sum |q_i p_i|            (4.7e-5 S)
//   accumulation in W    <= 17 * 2^-23 per matrix instruction, at most 13     (2.7e-5 S, allowing
//                           for truncating adds of every term)
// together below FILTER_REL = 2^-13 (1.22e-4) of S with a factor of 1.5 to spare.  The norm pieces
// (one share per group of 8 dimensions, each lowered and cut by itself and added up by the matrix
// instruction of the norm cell) hold at most N (1 - NORM_LOWER) (1 + 2^-15.3) (cutting, the sums of
// a share, one rounding), and NORM_LOWER = 2^-12 + 2^-14 >= 2 FILTER_REL + 2^-15.3, so that
//   W <= V + FILTER_REL * Q        whenever V is finite,
// and a pair can only have V < radius if W < radius + FILTER_REL * Q.  The compare is written so
// that a NaN in W passes; FILTER_ABS covers products of pieces that underflow.
// In 65 .. 128 dimensions (26 matrix instructions per tile, d + 2 <= 130 roundings in V) the three
// terms are 7.8e-6, 4.7e-5 and 5.3e-5 of S: FILTER_REL_WIDE = 1.5 * 2^-13 (1.83e-4) leaves a factor
// of 1.7, with NORM_LOWER_WIDE = 1.75 * 2^-12 >= 2 FILTER_REL_WIDE + 2^-15.3.
// In 129 .. 256 dimensions (FUSED_ARITH_EXACT_F32) W comes from v_mfma_f32_32x32x2_f32 on the plain
// values and on norm shares lowered by NORM_LOWER: at most 258 accumulations of 2^-23 each (3.1e-5 S),
// the shares' own sums (64 * 2^-24 N) and the d + 2 <= 258 roundings of V (1.5e-5 S), 5e-5 S together
// against FILTER_REL = 2^-13 (1.22e-4).
constexpr float FILTER_REL = 0x1.0p-13F;
constexpr float NORM_LOWER = 0x1.4p-12F;
constexpr float FILTER_REL_WIDE = 0x1.8p-13F;
constexpr float NORM_LOWER_WIDE = 0x1.cp-12F;
constexpr float FILTER_ABS = 0x1.0p-100F;
// norm of the points beyond the end of a range: the largest finite bf16, so that they only pass the
// filter while a radius is still infinite (what passes is checked against the range again)
constexpr u32 BF16_HUGE = 0x7F7FU;

// Stage geometry by padded dimension DP.
//
// SPLIT = false: fp32 matrix instructions; a stage is (DP + norm rows) x PT floats, PT points per
// stage so that it stays below 20 KB for DP <= 128.
//
// SPLIT = true (DP <= 64): every fp32 value x is cut into three bf16 pieces x = x1 + x2 + x3
// (exactly: 8 + 8 + 8 significant bits) and a product x*y is the sum of the bf16 products
// x3*y1 + x2*y2 + x1*y3 + x2*y1 + x1*y2 + x1*y1 accumulated in fp32 (what is left out is below
// 2^-23 of the product, the size of one fp32 rounding).  The bf16 matrix path runs at 16 times
// the fp32 one and does not share the vector unit with it.  A stage holds, per piece and per 8
// dimensions, one 16-byte cell per point (the A operand of v_mfma_f32_32x32x16_bf16), then the
// norms of the points.
// Per-query buffers: 32 slots, the points of one matrix tile.  Every merge pays for the whole list,
// so for lists of 128 entries and more the buffers can have 64 slots where the stages leave room
// for them (up to 16 dimensions, with smaller stages): half as many merges.  That pays where the
// lists hardly converge, i.e. with few queries whose points are cut into ranges (q = 8192,
// n = 2^17, d = 8: 4.4 -> 2.7 ms at k = 256 and 1.7 -> 1.3 ms at k = 128 before the first radii from
// a sample; at k = 64 the smaller stages cost more than the merges save).  WIDE_OK is set for
// launches over ranges only (see launch_fused).
constexpr int RING_MAX_DP = 256; // largest padded dimension that takes the ring of stages
constexpr int FQ_XCHG = 96;      // words a wave has for the exchange at a merge: 32 radii, fills, labels

template <int DP, int ARITH, int K, bool WIDE_OK = false, bool BIG_OK = false>
struct fused_geometry
{
    static constexpr bool SPLIT = ARITH == FUSED_ARITH_BF16X3;
    static constexpr bool EXACT = ARITH == FUSED_ARITH_EXACT;
    // BIG: workgroups of eight waves (256 queries) that share stages of twice the points, one
    // workgroup per compute unit -- the same two waves per SIMD, but half the staging, LDS writes
    // and hand-overs per pair.  The exact arithmetic in 32 dimensions on the ring of stages; worth
    // it where the queries alone give every compute unit such a workgroup (launch_fused).
    // (65 .. 128 dimensions exist in this shape only: a stage of 32 points has 34 KB there)
    static constexpr bool BIG = BIG_OK && ARITH == FUSED_ARITH_EXACT && DP <= 128;
    static constexpr int WAVES = BIG ? 2 * FQ_WAVES : FQ_WAVES;
    static constexpr int THREADS = WAVES * WAVE;
    static constexpr int QB = FQ_QW * WAVES; // queries per workgroup
    static constexpr bool WIDE = WIDE_OK && K >= 128 && DP <= 16 && ARITH == FUSED_ARITH_MFMA_F32;
    static constexpr int CAP = WIDE ? 2 * FQ_CAP : FQ_CAP; // buffer slots per query
    static constexpr int DK = DP < 16 ? 16 : DP;       // SPLIT, EXACT: dimensions padded to whole matrix steps
    static constexpr int KB = DK / 16;                 // SPLIT, EXACT: matrix steps of 16 dimensions
    static constexpr int KS = DK / 8;                  // SPLIT, EXACT: cells of 8 dimensions per point and piece
    // EXACT: a stage holds the points as fp32 rows (for the sequential arithmetic of what passes the
    // filter) and as 16-byte cells of bf16 pieces (the A operands of the filter's matrix
    // instructions): two pieces per value and a cell with two pieces of the lowered norm.  Up to 8
    // dimensions a point is three cells, (piece 1 | piece 2 | norm), used as the two halves of the
    // 16 matrix dimensions.
    // (one norm cell holds the shares of four groups of 8 dimensions: a second one where eight
    // groups are staged by eight waves, four for the sixteen groups of 128 dimensions)
    static constexpr int NORM_CELLS = DP == 128 && BIG ? 4 : (DP == 64 && BIG ? 2 : 1);
    static constexpr int CELLS = EXACT ? (DP <= 8 ? 3 : 2 * KS + NORM_CELLS) : 0;
    // matrix instructions that add up the norm cells: one takes a cell in the first half of its 16
    // inner dimensions (against ones there and zeros in the second half), or two cells, one in
    // either half (against ones throughout)
    static constexpr int NORM_TERMS = NORM_CELLS >= 2 ? NORM_CELLS / 2 : 1;
    static constexpr int PT = SPLIT   ? (DK <= 16 ? 128 : (DK <= 32 ? 64 : 32))
                              : EXACT ? (DP <= 16 ? 128 : (DP <= 32 ? 64 : (DP <= 64 ? 32 : 16))) * (BIG ? 2 : 1)
                              : WIDE  ? (DP <= 8 ? 128 : 64)
                                      : (DP <= 16 ? 256 : (DP <= 32 ? 128 : (DP <= 64 ? 64 : 32)));
    // threads per point when staging.  The small stages of the 64-slot geometry are staged by their
    // first PT threads, a whole point each, so that the norm of a point is one row and can be the
    // initial accumulator as in the 32-slot geometry (same terms in the same order: both
    // geometries give the same bits).  EXACT: a thread carries 8 consecutive dimensions of a point
    // (4 in up to 8 dimensions), as with bf16x3 products.
    static constexpr int TPP = EXACT ? THREADS / PT : (WIDE ? 1 : THREADS / PT);
    static constexpr int STAGERS = SPLIT ? THREADS : TPP * PT; // threads that stage
    // point rows (zero beyond dim), then one row per staging thread of a point with its share of
    // ||p||^2 (at least two rows, so that the row count is even)
    // (one row where it is read as the initial accumulator and never multiplied)
    // PAIRED: the 2 or 4 staging threads of a point are neighbouring lanes, which add up their
    // shares of the norm among themselves: one norm row, read as the initial accumulator
    // (not for lists of 128 entries in 32 dimensions: that instantiation then needs 260 vector
    // registers, 4 more than two waves per SIMD leave it)
    static constexpr bool PAIRED =
        !SPLIT && !EXACT && !WIDE && (TPP == 2 || TPP == 4) && PT >= 64 && !(DP == 32 && K == 128);
    static constexpr int NORM_ROWS = (!SPLIT && (TPP == 1 || PAIRED) && PT >= 64) ? 1 : (TPP > 2 ? TPP : 2);
    static constexpr int ROWS = DP + NORM_ROWS;
    static constexpr int STEPS = ROWS / 2;    // MFMA steps of 2 rows
    static constexpr int VPT = SPLIT ? 8 : DP / TPP; // values a thread carries from global memory to LDS
    // MFMA row tiles per stage; the exact arithmetic takes the stages of 256 points in two passes
    // of four tiles
    static constexpr int MT = EXACT && PT > 128 ? 4 : PT / 32;
    static constexpr int SUB = PT / 32 / MT;
    static constexpr int STAGE_FLOATS = SPLIT   ? 3 * KS * PT * 4 + PT
                                        : EXACT ? DP * PT + CELLS * PT * 4
                                                : ROWS * PT;
    // Stages in LDS: two, with a barrier per stage (one being multiplied, one being filled), or a
    // ring of three without barriers, in which a wave that appends or merges holds up the others
    // only once it is a whole stage behind (see the stage loop of the kernel).  Two workgroups per
    // compute unit have 80 KB of LDS each:
    //  * up to 8 dimensions three stages fit next to the query buffers.  Lists of 256 entries stay
    //    with the barrier: their merges are so long that the waves of a workgroup do better
    //    merging together, which leans on the barrier (65536 queries x 2^20 points, d = 8:
    //    k = 64 14.8 -> 13.9 ms, k = 128 16.4 -> 15.9 ms on the ring, k = 256 19.9 -> 21.9 ms);
    //  * in 16 to 128 dimensions a stage has 17 KB, and three fit if the query buffers give up a
    //    quarter of their slots (24 of 32: a few more merges).  Lists of up to 32 entries only:
    //    longer ones sort their buffers in place, all 32 slots of them, and with that changed they
    //    gain 2-3 % at k = 64 on many queries but lose 4-8 % (k = 64) and 26 % (k = 128) over
    //    ranges of points, where merges of long lists are what the time goes into.  (65536 queries x 2^20
    //    points, k = 32: d = 16 20.4 -> 19.9 ms, d = 32 38.5 -> 37.5 ms, d = 64 75.4 -> 73.0 ms,
    //    d = 128 138.7 -> 137.9 ms.)  In 256 dimensions, where a compute unit holds one workgroup
    //    anyway (registers), three stages of 33 KB: d = 256, k = 32 304 -> 283 ms; with longer lists
    //    it gains 4 % on many queries but loses a third over ranges (k = 256, 8192 x 2^17: 7.2 -> 9.9 ms).
    //  * the stages of the bf16 pieces have 12.5 KB in every dimension: three fit as they are.
    //    Lists of up to 32 entries (65536 queries x 2^20 points, k = 32: d = 16 14.0 -> 13.8 ms,
    //    d = 64 51.2 -> 47.0 ms; 8192 queries x 2^17 points over ranges: d = 16 0.78 -> 0.68 ms,
    //    d = 32 0.96 -> 0.87 ms); lists of 64 and 128 gain 4 % on many queries and lose 14 % over
    //    ranges.
    // (The geometry with 64-slot buffers would have room for three of its small stages, but its
    // long lists over ranges want the waves merging together: 8192 queries x 2^17 points, d = 8,
    // k = 128 1.10 -> 1.46 ms on the ring.)
    // (The workgroups of 256 queries have the LDS of a whole compute unit: the ring for every list
    // length, with buffers of 20 to 32 slots.  So has the exact arithmetic of 129 .. 256 dimensions,
    // one workgroup of four waves per compute unit, whose candidates differ most from wave to wave:
    // 65536 queries x 2^20 points, d = 256, k = 32: 452 -> 376 ms against the two stages with a barrier.)
    static constexpr bool RING =
        !WIDE && (SPLIT ? K <= FQ_CAP
                        : BIG || ARITH == FUSED_ARITH_EXACT_F32 || (DP <= 8 && K <= 128) ||
                              (DP >= 16 && DP <= RING_MAX_DP && K <= FQ_CAP));
    static constexpr int NB = RING ? 3 : 2;
    // slots a query buffer has in LDS (20 where the three stages of 256 points in 16 dimensions leave
    // no more room next to the buffers of 256 queries)
    static constexpr int SLOTS = EXACT && K <= 16 ? 16
                                 : BIG && DP == 16 ? 20
                                 : RING && !SPLIT && DP >= 16 ? 24
                                                              : CAP;
    // (lists longer than a buffer sort their buffers as CAP keys; a buffer of fewer slots keeps the
    // last SLOTS of them, since the first CAP - SLOTS of the descending order are padding)
    static constexpr int DROP = CAP - SLOTS;
    static_assert(!SPLIT || (DP <= 64 && TPP == KS), "one staging thread per point and cell");
    static_assert(!EXACT || ((DP <= 64 || (DP == 128 && BIG)) && VPT == (DP <= 8 ? 4 : 8) && MT <= 4 && SUB <= 2),
                  "the stages of the exact arithmetic serve up to 64 dimensions (128 in workgroups of 256 "
                  "queries), in passes of at most four tiles");
    static constexpr size_t lds_bytes()
    {
        // the stages, the query buffers, exchange slots, merge flags and stage counters
        return NB * static_cast<size_t>(STAGE_FLOATS) * sizeof(float) +
               static_cast<size_t>(WAVES) * FQ_QW * SLOTS * sizeof(u64) +
               static_cast<size_t>(WAVES) * FQ_XCHG * sizeof(float) + 8 * sizeof(int);
    }
    static_assert(!EXACT || lds_bytes() <= (BIG ? 160 : 80) * 1024, "two workgroups per compute unit, or one of eight waves");
};

// K: list length.  DP: dimension padded to 8, 16, 32, 64, 128 or 256 (padding rows are zero on
// both sides of the product).
template <int K, int DP, int ARITH, bool WIDE_OK, bool BIG_OK = false>
__global__ void __launch_bounds__((fused_geometry<DP, ARITH, K, WIDE_OK, BIG_OK>::THREADS)) fused_kernel(const fused_args a)
{
    using G = fused_geometry<DP, ARITH, K, WIDE_OK, BIG_OK>;
    constexpr int FQ_THREADS = G::THREADS; // (the workgroup's shape, which shadows the usual one)
    constexpr int FQ_WAVES = G::WAVES;
    constexpr int FQ_QB = G::QB;
    constexpr bool SPLIT = G::SPLIT;
    constexpr bool EXACT = G::EXACT;
    // 129 .. 256 dimensions of the default arithmetic: stages, matrix instructions and loops of the
    // fp32 kernel, whose values (on lowered norms) only filter; lists as with EXACT
    constexpr bool VIA_F32 = ARITH == FUSED_ARITH_EXACT_F32;
    constexpr bool EXACT_LISTS = EXACT || VIA_F32;
    static_assert(!VIA_F32 || (G::MT == 1 && !G::PAIRED), "one tile per stage, a norm row per staging thread");
    constexpr int PT = G::PT;
    constexpr int CAP = G::CAP;
    constexpr int SLOTS = G::SLOTS;
    constexpr int DROP = K > CAP ? G::DROP : 0;
    // Norms in the accumulator: where ||p||^2 is one row after the point rows -- one staging thread
    // carries a whole point (DP <= 16), or the 2 or 4 staging threads of a point are neighbouring
    // lanes that add up their shares (DP = 32, 64) -- it is read as the initial value of the
    // accumulators, which saves the matrix step that would add it (one of 5 at DP = 8, of 9 at 16,
    // of 17 at 32, of 33 at 64; 65536 queries x 2^20 points, k = 32: d = 32 37.7 -> 36.4 ms, d = 64
    // 73.0 -> 71.8 ms).  The sum then starts from the norm instead of ending with it: same terms,
    // another rounding order.
    constexpr bool NORM_IN_C = SPLIT || ((G::TPP == 1 || G::PAIRED) && G::MT >= 2);
    constexpr int STEPS = NORM_IN_C ? DP / 2 : G::STEPS;
    constexpr int KB = G::KB;
    constexpr int KS = G::KS;
    constexpr int TPP = G::TPP;
    constexpr int VPT = G::VPT;
    constexpr int MT = G::MT;
    // merge layout: S keys per query spread over LPQ lanes, R keys per lane
    constexpr int S = K > CAP ? K : CAP;
    constexpr int R = 4;
    constexpr int LPQ = S / R;
    constexpr int QPP = WAVE / LPQ;           // queries per merge pass
    constexpr int PASSES = FQ_QW / QPP;
    // Whether the waves of a workgroup merge together (below): pays for the long merges of long
    // lists (k = 256: 65 -> 52 ms); for k <= 32 the two looks at the flag per stage cost more (1 %
    // each) than the short merges they overlap.
    constexpr bool JOIN_MERGES = K > CAP && !G::RING;

    extern __shared__ float lds[];
    constexpr int STAGE_FLOATS = G::STAGE_FLOATS;
    float* const stages = lds;                                                    // [NB][STAGE_FLOATS]
    constexpr bool RING = G::RING;
    constexpr int NB = G::NB;
    u64* const buffers = reinterpret_cast<u64*>(lds + NB * STAGE_FLOATS);          // [waves][32][SLOTS]
    float* const xchg = reinterpret_cast<float*>(buffers + FQ_WAVES * FQ_QW * SLOTS);  // [waves][96]
    int* const merge_wanted = reinterpret_cast<int*>(xchg + FQ_WAVES * FQ_XCHG);        // [3]
    int* const ready = merge_wanted + 4;   // [3] waves that have written their part, per ring slot

    const int dim = a.dim;
    // this workgroup's range of points
    const int n_begin = static_cast<int>(blockIdx.y) * a.split_points;
    const int n = a.visit < n_begin + a.split_points ? a.visit : n_begin + a.split_points;
    const size_t total_points = static_cast<size_t>(a.n);
    const size_t list_stride = static_cast<size_t>(a.list_stride);
    const int t = static_cast<int>(threadIdx.x);
    const int lane = t & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(t / WAVE);
    const int half = lane / 32;               // which of the two rows of an MFMA step
    const int ql = lane & 31;                 // query of this lane inside the wave
    const int wave_q0 = static_cast<int>(blockIdx.x) * FQ_QB + wave * FQ_QW;
    const int my_q = wave_q0 + ql;
    u64* const wbuf = buffers + static_cast<size_t>(wave) * FQ_QW * SLOTS;
    float* const wx = xchg + wave * FQ_XCHG;  // 32 radii, then 32 fills (as int bits), then the
                                              // labels of the radii (EXACT)

    // query fragment: step s of this lane is row 2s + half, times -2 (the stages hold the plain
    // point values); the norm rows are multiplied by 1
    float qf[SPLIT || EXACT ? 1 : STEPS];
    // SPLIT: the three bf16 pieces of -2q for the 8 dimensions 16*kb + 8*half .. + 7 of step kb
    // EXACT: two pieces; up to 8 dimensions qs[0][0] is piece 1 of dimensions 0 .. 7 in both halves
    // of the wave and qs[1][0] piece 2 in the first half, (1, 1, 0, ...) for the norm cell in the
    // second; from 16 dimensions on qs[2][0] is the norm cell's (1, 1, 0, ...) in the first half
    // (ones in both halves where a point has two or four norm cells, which the halves take in pairs)
    vuint4 qs[SPLIT || EXACT ? 3 : 1][SPLIT || EXACT ? KB : 1];
    // EXACT: the query itself, every dimension, for the sequential arithmetic; the slack of its
    // filter threshold above the radius
    // (beyond 64 dimensions the query is read again where a candidate needs it)
    constexpr bool QUERY_IN_REGISTERS = EXACT && DP <= 64;
    constexpr float FILTER_REL_DP = DP > 64 ? FILTER_REL_WIDE : FILTER_REL;
    constexpr float NORM_LOWER_DP = DP > 64 ? NORM_LOWER_WIDE : NORM_LOWER;
    float qx[QUERY_IN_REGISTERS ? DP : 1];
    float filter_slack = 0.0F;
    float thr = __builtin_inff();    // EXACT: what a filter value must not exceed to be looked at
    int radius_label = 0x7FFFFFFF;   // EXACT: label of the list entry the radius comes from
    qx[0] = 0.0F;
    if constexpr (EXACT)
    {
        float qq = 0.0F;
        // (every load from a valid address, so that they are all in flight together)
        const bool live = my_q < a.q;
        const float* const mine = a.queries + (live ? my_q : 0);
        // (the norm cell holds two pieces per share of the norm, at most four shares)
        const vuint4 ones{0x3F803F80U, 0x3F803F80U, 0x3F803F80U, 0x3F803F80U};
        const vuint4 zeros{0, 0, 0, 0};
        if constexpr (QUERY_IN_REGISTERS)
        {
#pragma unroll
            for (int dd = 0; dd < DP; ++dd)
            {
                const float x = mine[static_cast<size_t>(dd < dim ? dd : 0) * a.q];
                qx[dd] = dd < dim && live ? x : 0.0F;
            }
#pragma unroll
            for (int dd = 0; dd < DP; ++dd)
            {
                qq = __builtin_fmaf(qx[dd], qx[dd], qq);
            }
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
            {
                float val[8];
#pragma unroll
                for (int j = 0; j < 8; ++j)
                {
                    // (a select between registers: the query is not indexed by the lane)
                    const int first = DP <= 8 ? j : 16 * kb + j;
                    const int second = DP <= 8 ? j : 16 * kb + 8 + j;
                    float lower = qx[first];
                    float upper = qx[second < DP ? second : 0];
                    asm volatile("" : "+v"(lower), "+v"(upper));
                    val[j] = -2.0F * (half != 0 ? upper : lower);
                }
                cut_bf16x2(val, qs[0][kb], qs[1][kb]);
                qs[2][kb] = half == 0 || G::NORM_CELLS >= 2 ? ones : zeros;
            }
        }
        else
        {
            // 16 dimensions at a time: the lane keeps the pieces of its half of them
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
            {
                float both[16];
#pragma unroll
                for (int j = 0; j < 16; ++j)
                {
                    const int dd = 16 * kb + j;
                    const float x = mine[static_cast<size_t>(dd < dim ? dd : 0) * a.q];
                    both[j] = dd < dim && live ? x : 0.0F;
                }
                float val[8];
#pragma unroll
                for (int j = 0; j < 16; ++j)
                {
                    qq = __builtin_fmaf(both[j], both[j], qq);
                }
#pragma unroll
                for (int j = 0; j < 8; ++j)
                {
                    float lower = both[j];
                    float upper = both[8 + j];
                    asm volatile("" : "+v"(lower), "+v"(upper));
                    val[j] = -2.0F * (half != 0 ? upper : lower);
                }
                cut_bf16x2(val, qs[0][kb], qs[1][kb]);
                qs[2][kb] = half == 0 || G::NORM_CELLS >= 2 ? ones : zeros;
            }
        }
        filter_slack = FILTER_REL_DP * qq * (1.0F + 0x1.0p-20F) + FILTER_ABS * (1.0F + qq);
        if constexpr (DP <= 8)
        {
            qs[1][0] = half == 0 ? qs[1][0] : ones;
        }
        qf[0] = 0.0F;
    }
    else if constexpr (SPLIT)
    {
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
        {
            float val[8];
#pragma unroll
            for (int j = 0; j < 8; ++j)
            {
                const int dd = 16 * kb + 8 * half + j;
                val[j] = 0.0F;
                if (dd < dim && my_q < a.q)
                {
                    val[j] = -2.0F * a.queries[static_cast<size_t>(dd) * a.q + my_q];
                }
            }
            split_bf16x3(val, qs[0][kb], qs[1][kb], qs[2][kb]);
        }
        qf[0] = 0.0F;
    }
    else
    {
        qs[0][0] = vuint4{0, 0, 0, 0};
#pragma unroll
        for (int s = 0; s < STEPS; ++s)
        {
            const int dd = 2 * s + half;
            float val = dd >= DP ? 1.0F : 0.0F;
            if (dd < dim && my_q < a.q)
            {
                val = -2.0F * a.queries[static_cast<size_t>(dd) * a.q + my_q];
            }
            qf[s] = val;
        }
        if constexpr (VIA_F32)
        {
            // ||q||^2 from the fragments (-2 q; a lane has every other dimension)
            float qq = 0.0F;
#pragma unroll
            for (int s = 0; s < STEPS; ++s)
            {
                const float half_of = 2 * s + half < DP ? -0.5F * qf[s] : 0.0F;
                qq = __builtin_fmaf(half_of, half_of, qq);
            }
            qq += __builtin_bit_cast(float, lane_xor32<32>(__builtin_bit_cast(u32, qq)));
            filter_slack = FILTER_REL * qq * (1.0F + 0x1.0p-20F) + FILTER_ABS * (1.0F + qq);
        }
    }

    // rows that never change in any stage: padding dimensions, unused norm rows
    for (int i = t; i < NB * STAGE_FLOATS; i += FQ_THREADS)
    {
        lds[i] = 0.0F;
    }
    if (t < 8)
    {
        merge_wanted[t] = 0;
    }
    __syncthreads();

    // A first radius from a launch over a sample of the points (FUSED_FIRST_RADIUS_FROM + rank):
    // what the filter drops is not below it, so the list of a query is exact if k of its distances
    // lie below its first radius.  With one range of points a query where they do not gets a NaN as
    // its k-th distance (no list holds one otherwise); with several ranges the lists of a range need
    // not fill up, and such a query shows as +inf at the end of its reduced list.  A further launch
    // (FUSED_REPEAT_MARKED) repeats the pass of the workgroups that have such a query from +inf;
    // all others leave at once.
    float first_radius = __builtin_inff();
    if (a.first_radius >= FUSED_FIRST_RADIUS_FROM && my_q < a.q)
    {
        first_radius = a.final_dist[static_cast<size_t>(my_q) * a.final_stride + (a.first_radius - FUSED_FIRST_RADIUS_FROM)];
    }
    if (a.first_radius == FUSED_REPEAT_MARKED)
    {
        // (negated compare: true for a NaN as well)
        const bool marked =
            my_q < a.q && !(a.final_dist[static_cast<size_t>(my_q) * a.final_stride + K - 1] < __builtin_inff());
        if (__syncthreads_or(marked ? 1 : 0) == 0)
        {
            return;
        }
    }
    // Lanes beyond the last query (the workgroup of a ragged end) take no candidates at all: with a
    // radius that stayed infinite they would take every point, and their wave would merge at every
    // tile (40000 queries x 2^20 points: 560 ms instead of 9).
    const bool live_query = my_q < a.q;
    float radius = live_query ? first_radius : -__builtin_inff(); // k-th smallest distance of my query so far
    if constexpr (EXACT_LISTS)
    {
        // (a first radius from a sample gives the filter its threshold from the first tile on)
        thr = live_query ? radius + (filter_slack + 0x1.0p-22F * __builtin_fabsf(radius)) : -__builtin_inff();
    }
    int fill = 0;                    // used slots of my query's buffer (same in both lanes of a query)
    bool have_list = false;          // wave-uniform: the lists in the output arrays are valid
    bool merged = false;             // wave-uniform: this wave has merged during the current stage
    int stage_slot = 0;              // stage index modulo 3: the slot of merge_wanted in use
    bool gave_up = false;            // wave-uniform: a wait for a stage of the ring ran out of polls
#ifdef BITSKNN_FUSED_TIMING
    long long ft_cycles[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    long long ft_mark = static_cast<long long>(__builtin_readcyclecounter());
#endif

    // ---- merge of all buffers of this wave into the lists --------------------------------------
    auto merge_event = [&]() __attribute__((always_inline)) {
        reinterpret_cast<int*>(wx)[32 + ql] = fill;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if constexpr (K > CAP)
        {
            // Lists longer than a buffer: the buffers are sorted in place first, 8 queries at a
            // time, so that the passes below only pay for the merge network of the list.
            constexpr int BR = 4;           // keys per lane
            constexpr int BL = CAP / BR; // lanes per buffer
#pragma unroll 1
            for (int pass = 0; pass < FQ_QW / (WAVE / BL); ++pass)
            {
                const int qm = pass * (WAVE / BL) + lane / BL;
                const int sub = lane % BL;
                const int used = reinterpret_cast<const int*>(wx)[32 + qm];
                u64 buf[BR];
#pragma unroll
                for (int r = 0; r < BR; ++r)
                {
                    const int i = sub * BR + r;
                    buf[r] = i < used ? wbuf[qm * SLOTS + i] : PAD_KEY;
                }
                net_sort<BL, BR, 2, true>(buf, nullptr, sub);
#pragma unroll
                for (int r = 0; r < BR; ++r)
                {
                    // (descending, padding first: at least the first DROP keys are padding)
                    const int i = sub * BR + r;
                    if (DROP == 0 || i >= DROP)
                    {
                        wbuf[qm * SLOTS + i - DROP] = buf[r];
                    }
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
        // The list of a query is read by the lanes that wrote it in the previous merge (same
        // pass, same positions), so plain loads and stores in program order are enough.  The list
        // of the next pass is requested before the network of this one runs.
        const int sub = lane % LPQ;
        float next_dist[R];
        std::int32_t next_label[R];
        auto request_list = [&](int pass) __attribute__((always_inline)) {
            const int gq = wave_q0 + pass * QPP + lane / LPQ;
            const size_t at = (static_cast<size_t>(gq) * a.splits + blockIdx.y) * list_stride + sub * R;
#pragma unroll
            for (int r = 0; r < R; ++r)
            {
                next_dist[r] = __builtin_inff();
                next_label[r] = 0x7FFFFFFF;
                if (have_list && sub * R + r < K && gq < a.q)
                {
                    next_dist[r] = a.out_dist[at + r];
                    next_label[r] = a.out_label[at + r];
                }
            }
        };
        request_list(0);
#pragma unroll 1
        for (int pass = 0; pass < PASSES; ++pass)
        {
            const int qm = pass * QPP + lane / LPQ; // query (inside the wave) of this lane group
            const int gq = wave_q0 + qm;
            const int used = reinterpret_cast<const int*>(wx)[32 + qm];
            u64 buf[R];
            u64 list[R];
#pragma unroll
            for (int r = 0; r < R; ++r)
            {
                const int i = sub * R + r;
                if constexpr (K > CAP)
                {
                    // the sorted buffer (descending, padding first) is the tail of a descending
                    // sequence of K keys
                    buf[r] = i >= K - CAP + DROP ? wbuf[qm * SLOTS + i - (K - CAP) - DROP] : PAD_KEY;
                }
                else
                {
                    buf[r] = i < used ? wbuf[qm * SLOTS + (i < SLOTS ? i : 0)] : PAD_KEY;
                }
                list[r] = make_key(next_dist[r], next_label[r]);
            }
            if (pass + 1 < PASSES)
            {
                request_list(pass + 1);
            }
            // buffer descending, element-wise minimum with the ascending list, re-sort
            if constexpr (K <= CAP)
            {
                net_sort<LPQ, R, 2, true>(buf, nullptr, sub);
            }
#pragma unroll
            for (int r = 0; r < R; ++r)
            {
                list[r] = buf[r] < list[r] ? buf[r] : list[r];
            }
            net_phase<LPQ, R, S, S / 2, false>(list, nullptr, sub);
#pragma unroll
            for (int r = 0; r < R; ++r)
            {
                const int i = sub * R + r;
                if (i < K && gq < a.q)
                {
                    const size_t at = (static_cast<size_t>(gq) * a.splits + blockIdx.y) * list_stride + i;
                    a.out_dist[at] = key_value(list[r]);
                    a.out_label[at] = key_label(list[r]);
                }
                if (i == K - 1)
                {
                    wx[qm] = key_value(list[r]);
                    if constexpr (EXACT_LISTS)
                    {
                        reinterpret_cast<int*>(wx)[64 + qm] = key_label(list[r]);
                    }
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // (a first radius from a sample stays until the list has a smaller one)
        radius = live_query ? fminf(wx[ql], first_radius) : -__builtin_inff();
        if constexpr (EXACT_LISTS)
        {
            // (the slack also covers the rounding of this sum)
            thr = live_query ? radius + (filter_slack + 0x1.0p-22F * __builtin_fabsf(radius)) : -__builtin_inff();
            // a value equal to the radius passes if its label is below the label of the list's last
            // entry (every label where the radius is a first radius from a sample)
            radius_label = wx[ql] < first_radius ? reinterpret_cast<const int*>(wx)[64 + ql] : 0x7FFFFFFF;
        }
        fill = 0;
        have_list = true;
        merged = true;
    };

    // position of this lane's A operands inside a stage row, for the two tiles of a pair (the
    // second one is kept opaque so that it stays a base register of its own)
    int tile_at[2] = {half * PT + ql, half * PT + ql + 32};
    asm volatile("" : "+v"(tile_at[1]));

    // ---- filter one 32 x 32 tile held in `acc` and append what passes ---------------------------
    // lane holds 16 distances of query ql: rows 8*(r/4) + 4*half + r%4 of the tile
    auto append_tile = [&](const vfloat16& acc, int tile_base) __attribute__((always_inline)) {
        // One compare per value: its lane mask stays in scalar registers and serves the count and
        // the predicate of the write (vector instructions take their cycles from the matrix
        // instructions of both waves of the SIMD, scalar ones do not).
        u64 pass[16];
        auto compare = [&]() __attribute__((always_inline)) -> int {
            int count = 0;
#pragma unroll
            for (int r = 0; r < 16; ++r)
            {
                const bool below = acc[r] < radius;
                pass[r] = __builtin_amdgcn_ballot_w64(below);
                count += below ? 1 : 0;
            }
            return count;
        };
        // the same for the values FROM..TO-1 of every lane only
        auto compare_some = [&](auto from_tag, auto to_tag) __attribute__((always_inline)) -> int {
            constexpr int FROM = decltype(from_tag)::value;
            constexpr int TO = decltype(to_tag)::value;
            int count = 0;
#pragma unroll
            for (int r = 0; r < 16; ++r)
            {
                pass[r] = 0;
                if (r >= FROM && r < TO)
                {
                    const bool below = acc[r] < radius;
                    pass[r] = __builtin_amdgcn_ballot_w64(below);
                    count += below ? 1 : 0;
                }
            }
            return count;
        };
        const int first_point = tile_base + 4 * half;
        // Most values of a tile that has candidates fail in every lane: they are skipped four at a
        // time (a taken branch costs a wave far more than one that is not; 16 of them per tile were
        // 2-4 % of the kernel time where candidates are rare).  The writes stay in line: moved out
        // of line they gain another 0.5 % there, but cost 3-7 % where most tiles hold candidates
        // (lists over ranges of points, which hardly converge).
        auto write = [&](int mine, int other) __attribute__((always_inline)) {
            int slot = fill + (half != 0 ? other : 0);
#pragma unroll
            for (int g = 0; g < 4; ++g)
            {
                if ((pass[4 * g] | pass[4 * g + 1] | pass[4 * g + 2] | pass[4 * g + 3]) != 0)
                {
#pragma unroll
                    for (int r = 4 * g; r < 4 * g + 4; ++r)
                    {
                        if (pass[r] != 0)
                        {
                            if (__builtin_amdgcn_inverse_ballot_w64(pass[r]))
                            {
                                wbuf[ql * SLOTS + slot] = make_key(acc[r], first_point + 8 * (r / 4) + (r % 4));
                                ++slot;
                            }
                        }
                    }
                }
            }
            fill += mine + other;
        };
        int mine = compare();
        int other = static_cast<int>(lane_xor32<32>(static_cast<u32>(mine)));
        if (__builtin_amdgcn_ballot_w64(fill + mine + other > SLOTS) != 0)
        {
            // the other waves of the workgroup would wait for this wave at the stage barrier:
            // they are asked to merge their buffers in the meantime
            if (JOIN_MERGES && lane == 0)
            {
                __hip_atomic_store(merge_wanted + stage_slot, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
            merge_event();
            mine = compare();
            other = static_cast<int>(lane_xor32<32>(static_cast<u32>(mine)));
            if constexpr (SLOTS < FQ_CAP)
            {
                // A tile can bring 32 candidates to a query (16 per lane), more than such a buffer
                // holds: a tile that does not fit the empty buffers is taken in two halves of 8
                // values per lane, with a merge in between.
                static_assert(SLOTS >= 16, "half a tile fits an empty buffer");
                if (__builtin_amdgcn_ballot_w64(mine + other > SLOTS) != 0)
                {
                    using std::integral_constant;
                    mine = compare_some(integral_constant<int, 0>{}, integral_constant<int, 8>{});
                    other = static_cast<int>(lane_xor32<32>(static_cast<u32>(mine)));
                    write(mine, other);
                    merge_event();
                    mine = compare_some(integral_constant<int, 8>{}, integral_constant<int, 16>{});
                    other = static_cast<int>(lane_xor32<32>(static_cast<u32>(mine)));
                }
            }
        }
        write(mine, other);
    };
    auto filter_tile = [&](const vfloat16& acc, int tile_base) __attribute__((always_inline)) {
        // The first read of the tile is a compare the compiler sees, so that it places the wait
        // states a matrix result needs before them; the minimum of the other 15 values is written
        // out as v_min3 (fminf would first quieten each operand with an instruction of its own),
        // and assembly operands are not covered by that hazard handling.
        const u64 last_passes = __builtin_amdgcn_ballot_w64(acc[15] < radius);
        __builtin_amdgcn_sched_barrier(0);
        float low[5];
#pragma unroll
        for (int g = 0; g < 5; ++g)
        {
            low[g] = min3(acc[3 * g], acc[3 * g + 1], acc[3 * g + 2]);
        }
        const float smallest = min3(min3(low[0], low[1], low[2]), low[3], low[4]);
        if ((last_passes | __builtin_amdgcn_ballot_w64(smallest < radius)) != 0)
        {
            append_tile(acc, tile_base);
        }
    };

    // ---- staging: global -> registers -> LDS ---------------------------------------------------
    // thread t carries dimensions (t / PT) + TPP*i of point t % PT, writes them as rows of the
    // stage and adds up its share of ||p||^2 (the shares of a point meet inside the MFMA)
    // PAIRED: thread t carries dimensions (t % TPP) + TPP*i of point t / TPP: the threads of a point
    // are neighbouring lanes, which add up their shares of the norm among themselves
    // SPLIT: thread t carries the 8 dimensions 8*(t % TPP) .. + 7 of point t / TPP (neighbouring
    // lanes as well)
    // EXACT: thread t carries the VPT dimensions VPT * (t / PT) .. of point t % PT, so that the
    // threads of a wave write neighbouring words, rows and cells of a stage (no two of them meet in
    // a bank of LDS); every group of VPT dimensions has its own share of the norm
    const int sp = EXACT ? t % PT : (SPLIT || G::PAIRED ? t / TPP : t % PT);
    const int sd0 = EXACT ? VPT * (t / PT) : (SPLIT ? VPT * (t % TPP) : (G::PAIRED ? t % TPP : t / PT));
    // EXACT: the word of a point's norm cell that takes this thread's share of the norm
    // (64 dimensions in workgroups of four waves: the two groups of a wave share a word)
    constexpr bool PAIRED_SHARES = DP == 64 && !G::BIG;
    const int norm_slot = PAIRED_SHARES ? wave : t / PT;
    auto dim_of = [&](int i) -> int { return SPLIT || EXACT ? sd0 + i : sd0 + TPP * i; };
    float pre[VPT];
    // Point values are read with buffer loads: a constant byte offset per value and lane (beyond
    // the resource for dimensions dim .. DP-1, which then read as zero; the hardware checks the
    // lane offset only) plus the scalar offset of the stage, so that a load needs no vector
    // arithmetic.  Point matrices of 2 GiB and more take the plain loads.
    const bool small_points = static_cast<size_t>(dim) * total_points * sizeof(float) < (1ULL << 31);
    const auto point_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(a.points), 0,
        small_points ? static_cast<int>(static_cast<size_t>(dim) * total_points * sizeof(float)) : 0, 0x00020000);
    constexpr int OUTSIDE = 0x7FFFFFF0;
    int load_off[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i)
    {
        const int dd = dim_of(i);
        load_off[i] = dd < dim && small_points
                          ? static_cast<int>((static_cast<size_t>(dd) * total_points + sp) * sizeof(float))
                          : OUTSIDE;
    }
    auto fetch = [&](int base) {
        if constexpr (G::STAGERS < FQ_THREADS)
        {
            if (t >= G::STAGERS) // (whole waves)
            {
                return;
            }
        }
        // first point of the stage in the matrix (a sample visits every sample_scale-th stage)
        const int at = base * a.sample_scale + a.sample_offset;
        if (small_points)
        {
            const int stage_off = at * static_cast<int>(sizeof(float));
            if (base + PT <= n)
            {
#pragma unroll
                for (int i = 0; i < VPT; ++i)
                {
                    pre[i] = __builtin_bit_cast(
                        float, __builtin_amdgcn_raw_buffer_load_b32(point_rsrc, load_off[i], stage_off, 0));
                }
            }
            else
            {
                // ragged last stage: points from n on read as zero
                const bool inside = base + sp < n;
#pragma unroll
                for (int i = 0; i < VPT; ++i)
                {
                    pre[i] = __builtin_bit_cast(
                        float, __builtin_amdgcn_raw_buffer_load_b32(point_rsrc, inside ? load_off[i] : OUTSIDE,
                                                                    stage_off, 0));
                }
            }
        }
        else
        {
            const int j = at + sp;
#pragma unroll
            for (int i = 0; i < VPT; ++i)
            {
                const int dd = dim_of(i);
                pre[i] = 0.0F;
                if (dd < dim && base + sp < n)
                {
                    pre[i] = a.points[static_cast<size_t>(dd) * total_points + j];
                }
            }
        }
    };
    // EXACT with a stage image (fused_args::image): the stages as they stand in LDS were written to
    // global memory by fused_image_kernel, one after the other; staging is then a copy of 16-byte
    // units, IU per thread, through registers -- no arithmetic in this kernel.
    constexpr int UNITS = EXACT ? STAGE_FLOATS / 4 : 1;
    constexpr int IU = EXACT ? (UNITS + FQ_THREADS - 1) / FQ_THREADS : 1;
    vuint4 img[IU];
    int img_off[IU];
    const auto image_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<void*>(EXACT ? a.image : nullptr), 0, EXACT ? a.image_bytes : 0, 0x00020000);
#pragma unroll
    for (int j = 0; j < IU; ++j)
    {
        img[j] = vuint4{0, 0, 0, 0};
        img_off[j] = t + FQ_THREADS * j < UNITS ? (t + FQ_THREADS * j) * 16 : OUTSIDE;
    }
    // (base is a multiple of PT, and so is the offset of a sample; beyond the image the loads read zero)
    auto fetch_image = [&](int base) __attribute__((always_inline)) {
        const int stage_off = (base * a.sample_scale + a.sample_offset) * (STAGE_FLOATS * 4 / PT);
#pragma unroll
        for (int j = 0; j < IU; ++j)
        {
            img[j] = __builtin_bit_cast(vuint4, __builtin_amdgcn_raw_buffer_load_b128(image_rsrc, img_off[j], stage_off, 0));
        }
    };
    auto deposit_image_unit = [&](float* stage, auto j_tag) __attribute__((always_inline)) {
        constexpr int j = decltype(j_tag)::value;
        if (FQ_THREADS * (j + 1) <= UNITS || t + FQ_THREADS * j < UNITS)
        {
            reinterpret_cast<vuint4*>(stage)[t + FQ_THREADS * j] = img[j];
        }
    };
    auto deposit = [&](float* stage, int base) {
        if constexpr (G::STAGERS < FQ_THREADS)
        {
            if (t >= G::STAGERS)
            {
                return;
            }
        }
        float share = 0.0F;
        if constexpr (EXACT)
        {
            // fp32 rows for the sequential arithmetic, then the cells of bf16 pieces
            float eight[8];
#pragma unroll
            for (int i = 0; i < 8; ++i)
            {
                eight[i] = i < VPT ? pre[i < VPT ? i : 0] : 0.0F;
            }
            vuint4 piece[2];
            cut_bf16x2(eight, piece[0], piece[1]);
#pragma unroll
            for (int i = 0; i < VPT; ++i)
            {
                share = __builtin_fmaf(pre[i], pre[i], share);
                stage[(sd0 + i) * PT + sp] = pre[i];
            }
            constexpr int PIECE2 = DP <= 8 ? 1 : KS; // first cell of the second pieces
            if constexpr (VPT == 8)
            {
                // (the cell of dimension group t / PT of point t % PT is cell t)
                vuint4* const cells = reinterpret_cast<vuint4*>(stage + DP * PT);
                cells[t] = piece[0];
                cells[PIECE2 * PT + t] = piece[1];
            }
            else
            {
                // half a cell per thread
                typedef u32 vuint2 __attribute__((ext_vector_type(2)));
                vuint2* const halves = reinterpret_cast<vuint2*>(stage + DP * PT);
                const int h = sd0 / 4;
                halves[2 * sp + h] = vuint2{piece[0][0], piece[0][1]};
                halves[2 * (PIECE2 * PT + sp) + h] = vuint2{piece[1][0], piece[1][1]};
            }
            if constexpr (PAIRED_SHARES)
            {
                // two groups of dimensions per wave: one share
                share += __builtin_bit_cast(float, lane_xor32<32>(__builtin_bit_cast(u32, share)));
            }
            {
                // the lowered share of the norm in two pieces, one word of the point's norm cell per
                // share (the matrix instruction adds them up); points beyond the end only pass an
                // infinite radius
                const float lowered = __builtin_fmaf(-NORM_LOWER_DP, share, share);
                const vfloat2 whole{lowered, 0.0F};
                const u32 first = __builtin_bit_cast(u32, __builtin_convertvector(whole, vbf16x2)) & 0xFFFFU;
                const vfloat2 rest{lowered - __builtin_bit_cast(float, first << 16U), 0.0F};
                const u32 second = __builtin_bit_cast(u32, __builtin_convertvector(rest, vbf16x2)) & 0xFFFFU;
                u32* const norm_cell =
                    reinterpret_cast<u32*>(reinterpret_cast<vuint4*>(stage + DP * PT) +
                                           (G::CELLS - G::NORM_CELLS + norm_slot / 4) * PT + sp);
                norm_cell[norm_slot % 4] = base + sp < n ? first | (second << 16U) : BF16_HUGE;
            }
        }
        else if constexpr (SPLIT)
        {
#pragma unroll
            for (int i = 0; i < 8; ++i)
            {
                share = __builtin_fmaf(pre[i], pre[i], share);
            }
            vuint4 piece[3];
            split_bf16x3(pre, piece[0], piece[1], piece[2]);
            vuint4* const cells = reinterpret_cast<vuint4*>(stage);
            const int ks = sd0 / 8;
#pragma unroll
            for (int c = 0; c < 3; ++c)
            {
                cells[(c * KS + ks) * PT + sp] = piece[c];
            }
            // the threads of a point are TPP neighbouring lanes
            share += __builtin_bit_cast(float, lane_xor32<1>(__builtin_bit_cast(u32, share)));
            if constexpr (TPP >= 4)
            {
                share += __builtin_bit_cast(float, lane_xor32<2>(__builtin_bit_cast(u32, share)));
            }
            if constexpr (TPP == 8)
            {
                share += __builtin_bit_cast(float, lane_xor32<4>(__builtin_bit_cast(u32, share)));
            }
            // points beyond the end get an infinite distance and never pass the filter
            stage[3 * KS * PT * 4 + sp] = base + sp < n ? share : __builtin_inff();
        }
        else
        {
#pragma unroll
            for (int i = 0; i < VPT; ++i)
            {
                const int dd = sd0 + TPP * i;
                share = __builtin_fmaf(pre[i], pre[i], share);
                // (dimensions from dim on were read as zero: their rows stay zero)
                stage[dd * PT + sp] = pre[i];
            }
            // points beyond the end get an infinite distance and never pass the filter
            // (with one staging thread per point the share is the norm, in row DP)
            if constexpr (G::PAIRED)
            {
                share += __builtin_bit_cast(float, lane_xor32<1>(__builtin_bit_cast(u32, share)));
                if constexpr (TPP == 4)
                {
                    share += __builtin_bit_cast(float, lane_xor32<2>(__builtin_bit_cast(u32, share)));
                }
                stage[DP * PT + sp] = base + sp < n ? share : __builtin_inff();
            }
            else
            {
                if constexpr (VIA_F32)
                {
                    // (the filter's norm: lowered by the error budget, as the bf16 filter's is)
                    share = __builtin_fmaf(-NORM_LOWER, share, share);
                }
                stage[(DP + sd0) * PT + sp] = base + sp < n ? share : __builtin_inff();
            }
        }
    };

    // ---- EXACT: the candidates of a stage.  `cand` has bit 16 * tile + r set where filter value r
    // of this lane in that tile of the stage is not above the lane's threshold.  Every lane works
    // through its own bits, lowest first: it computes the distance of its query to that point with
    // sequential fused multiply-adds over the dimensions in order -- norm and dot product, then
    // norm - 2 dot: the reference's arithmetic (include/bits/topk/singlepass/
    // fused_cache_kernel_structs.cuh:457-522, :622-631) -- and appends it if its key is below the
    // key of the list's last entry.  (The full key: the lanes of a query take its points out of
    // index order, and a merge may fall between two of them.)  `base` is the stage's first point.
    auto exact_candidates = [&](u64 cand, const float* stage, int base) __attribute__((always_inline)) {
        while (__builtin_amdgcn_ballot_w64(cand != 0) != 0)
        {
            // an iteration brings a query at most two values
            if (__builtin_amdgcn_ballot_w64(fill + 2 > SLOTS) != 0)
            {
                if (JOIN_MERGES && lane == 0)
                {
                    __hip_atomic_store(merge_wanted + stage_slot, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                }
                merge_event();
            }
            const bool has = cand != 0;
            const int r = has ? __builtin_ctzll(cand) : 0;
            cand &= cand - 1;
            const int local = 32 * (r >> 4) + 8 * ((r >> 2) & 3) + 4 * half + (r & 3);
            const float* const column = stage + local;
            float norm = 0.0F;
            float dot = 0.0F;
            if constexpr (QUERY_IN_REGISTERS)
            {
#pragma unroll
                for (int dd = 0; dd < DP; ++dd)
                {
                    const float x = column[dd * PT];
                    norm = __builtin_fmaf(x, x, norm);
                    dot = __builtin_fmaf(qx[dd], x, dot);
                }
            }
            else if constexpr (VIA_F32)
            {
                // the query from the fragments of the matrix instructions (-2 q, halved exactly): a
                // lane has every other dimension, the lane of the other half of the wave, which
                // has the same query, the ones in between
                static_for<0, DP / 32>([&](auto c_tag) {
                    constexpr int c = decltype(c_tag)::value;
                    if (32 * c < dim)
                    {
#pragma unroll
                        for (int s = 16 * c; s < 16 * c + 16; ++s)
                        {
                            const u32 bits = __builtin_bit_cast(u32, qf[s]);
                            const auto both = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
                            // (copied out before the cast: a cast of an element of a vector reads
                            // the vector's first element with this compiler)
                            const u32 of_first_half = both[0];
                            const u32 of_second_half = both[1];
                            const float even = -0.5F * __builtin_bit_cast(float, of_first_half);
                            const float odd = -0.5F * __builtin_bit_cast(float, of_second_half);
                            const float x0 = column[(2 * s) * PT];
                            const float x1 = column[(2 * s + 1) * PT];
                            norm = __builtin_fmaf(x0, x0, norm);
                            dot = __builtin_fmaf(even, x0, dot);
                            norm = __builtin_fmaf(x1, x1, norm);
                            dot = __builtin_fmaf(odd, x1, dot);
                        }
                    }
                });
            }
            else
            {
                // the query comes from memory again, QC dimensions at a time, whose loads are all
                // issued ahead of their arithmetic (zero beyond dim, as the point's rows are; the
                // dimensions from dim on add nothing to either sum and are left out).  The two
                // halves of the wave have the same queries: of every 16 dimensions each half loads
                // 8 and a swap of the halves hands them to the other.
                constexpr int QC = 32;
                const float* const mine_first = a.queries + (my_q < a.q ? my_q : 0);
                const float* const mine = mine_first + static_cast<size_t>(8 * half) * static_cast<size_t>(a.q);
#pragma unroll 1
                for (int d0 = 0; d0 < dim; d0 += QC)
                {
                    float y[QC];
                    float mine_of[QC / 2];
                    if (d0 + QC <= dim)
                    {
#pragma unroll
                        for (int j = 0; j < QC / 2; ++j)
                        {
                            mine_of[j] = mine[static_cast<size_t>(d0 + 16 * (j / 8) + j % 8) * a.q];
                        }
                    }
                    else
                    {
#pragma unroll
                        for (int j = 0; j < QC / 2; ++j)
                        {
                            // (the first half's dimension `at`, the second half's at + 8: every
                            // lane loads from a row that exists, by an index the wave shares)
                            const int at = d0 + 16 * (j / 8) + j % 8;
                            const bool first_inside = at < dim;
                            const bool second_inside = at + 8 < dim;
                            const float* const from = second_inside ? mine : mine_first;
                            const float there = from[static_cast<size_t>(first_inside ? at : 0) * a.q];
                            mine_of[j] = (half == 0 ? first_inside : second_inside) ? there : 0.0F;
                        }
                    }
#pragma unroll
                    for (int j = 0; j < QC / 2; ++j)
                    {
                        const u32 bits = __builtin_bit_cast(u32, mine_of[j]);
                        const auto both = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
                        // (copied out before the cast: a cast of an element of a vector reads the
                        // vector's first element with this compiler)
                        const u32 of_first_half = both[0];
                        const u32 of_second_half = both[1];
                        y[16 * (j / 8) + j % 8] = __builtin_bit_cast(float, of_first_half);
                        y[16 * (j / 8) + 8 + j % 8] = __builtin_bit_cast(float, of_second_half);
                    }
#pragma unroll
                    for (int j = 0; j < QC; ++j)
                    {
                        const float x = column[(d0 + j) * PT];
                        norm = __builtin_fmaf(x, x, norm);
                        dot = __builtin_fmaf(y[j], x, dot);
                    }
                }
            }
            const float value = __builtin_fmaf(-2.0F, dot, norm);
            const int label = base + local;
            const bool below = has && label < n && (value < radius || (value == radius && label < radius_label));
            const u64 pass = __builtin_amdgcn_ballot_w64(below);
            if (pass != 0)
            {
                const int mine = below ? 1 : 0;
                const int other = static_cast<int>((pass >> (static_cast<unsigned>(lane) ^ 32U)) & 1U);
                if (below)
                {
                    wbuf[ql * SLOTS + fill + (half != 0 ? other : 0)] = make_key(value, label);
                }
                fill += mine + other;
            }
        }
    };
    // the filter of a tile: the smallest of the 16 values of every lane (a NaN if there is one),
    // eight v_minimum3_f32
    auto smallest_of = [&](const vfloat16& w) __attribute__((always_inline)) -> float {
        auto least = [](float a, float b, float c) __attribute__((always_inline)) -> float {
            return __builtin_elementwise_minimum(__builtin_elementwise_minimum(a, b), c);
        };
        float low[5];
#pragma unroll
        for (int g = 0; g < 5; ++g)
        {
            low[g] = least(w[3 * g], w[3 * g + 1], w[3 * g + 2]);
        }
        const float upper = least(low[3], low[4], w[15]);
        return __builtin_elementwise_minimum(least(low[0], low[1], low[2]), upper);
    };
    // bit r where value r of this lane is not above the threshold (negated compare: a NaN counts)
    auto bits_of = [&](const vfloat16& w) __attribute__((always_inline)) -> u32 {
        // two instructions per value: the compare, then bits = 2 bits + its result as the carry
        u32 bits = 0;
#pragma unroll
        for (int r = 15; r >= 0; --r)
        {
            asm("v_cmp_ngt_f32 vcc, %1, %2\n\tv_addc_co_u32 %0, vcc, %0, %0, vcc"
                : "+v"(bits)
                : "v"(w[r]), "v"(thr)
                : "vcc");
        }
        return bits;
    };

    // EXACT, first half of a stage: the filter values of all its tiles, lowered norm - 2 q.p from the
    // pieces.  The matrix instructions of the tiles take turns, term by term, so that none waits for
    // the result of the one before it.
    auto filter_values = [&](const float* stage, vfloat16 (&w)[MT]) __attribute__((always_inline)) {
        const vuint4* const cells = reinterpret_cast<const vuint4*>(stage + DP * PT);
        vfloat16 zero;
#pragma unroll
        for (int r = 0; r < 16; ++r)
        {
            zero[r] = 0.0F;
        }
        constexpr int TERMS = DP <= 8 ? 2 : 3 * KB + 1;
        vuint4 cell[MT][DP <= 8 ? 2 : 2 * KB + 1];
#pragma unroll
        for (int t = 0; t < MT; ++t)
        {
            const vuint4* const mine = cells + 32 * t + ql;
            if constexpr (DP <= 8)
            {
                // first half of the wave: piece 1 of the point against pieces 1 and 2 of the query;
                // second half: piece 2 against piece 1, the norm cell against (1, 1)
                cell[t][0] = mine[(half != 0 ? 1 : 0) * PT];
                cell[t][1] = mine[(half != 0 ? 2 : 0) * PT];
            }
            else
            {
#pragma unroll
                for (int kb = 0; kb < KB; ++kb)
                {
                    cell[t][kb] = mine[(2 * kb + half) * PT];
                    cell[t][KB + kb] = mine[(KS + 2 * kb + half) * PT];
                }
                cell[t][2 * KB] = mine[2 * KS * PT];
            }
        }
        static_for<0, TERMS>([&](auto j_tag) {
            constexpr int j = decltype(j_tag)::value;
            // term j: which cell of the point against which operand of the query (up to 8
            // dimensions: the two cells in turn; else per 16 dimensions piece 2 x piece 1,
            // piece 1 x piece 2, piece 1 x piece 1, and the norm cell last)
            constexpr bool norm_term = DP > 8 && j == 3 * KB;
            constexpr int kb = DP <= 8 || norm_term ? 0 : j / 3;
            constexpr int which = DP <= 8 ? j : j % 3;
            constexpr int a_at = DP <= 8 ? j : (norm_term ? 2 * KB : (which == 0 ? KB + kb : kb));
            constexpr int b_piece = DP <= 8 ? j : (norm_term ? 2 : (which == 1 ? 1 : 0));
            constexpr int b_kb = kb;
#pragma unroll
            for (int t = 0; t < MT; ++t)
            {
                w[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                    __builtin_bit_cast(vbf16x8, cell[t][a_at]), __builtin_bit_cast(vbf16x8, qs[b_piece][b_kb]),
                    j == 0 ? zero : w[t], 0, 0, 0);
            }
        });
    };
    // EXACT: the filter values of a stage as above, with the cutting of the values in `pre` (a stage
    // further on) into bf16 pieces placed between the matrix instructions, a few vector instructions
    // after each of the first ones, where they execute next to it; scheduling barriers keep the
    // order written here.  The pieces stay in registers (cut1, cut2, cut_norm) until write_cut puts
    // them into a stage.  `cut_base`: first point of the stage the values belong to.  MODE 2 (stages
    // from an image): nothing to cut.
    u32 cut1[4] = {0, 0, 0, 0};
    u32 cut2[4] = {0, 0, 0, 0};
    u32 cut_norm = 0;
    constexpr int NCELL = DP <= 8 ? 2 : 2 * KB + G::NORM_TERMS; // cells of a point that a lane reads
    // the tiles of a stage are multiplied in groups whose cells fit into 48 registers
    constexpr int TG = MT * NCELL <= 12 ? MT : (2 * NCELL <= 12 ? 2 : 1);
    // (the cells are read in the order in which the matrix instructions take them, the norm cell
    // last, so that the first instruction waits for the first read only)
    auto read_cells = [&](const float* stage, vuint4 (&cell)[TG][NCELL], int first_tile) __attribute__((always_inline)) {
        const vuint4* const cells = reinterpret_cast<const vuint4*>(stage + DP * PT);
        const vuint4* const mine = cells + 32 * first_tile + ql;
        if constexpr (DP <= 8)
        {
#pragma unroll
            for (int c = 0; c < 2; ++c)
            {
#pragma unroll
                for (int t = 0; t < TG; ++t)
                {
                    cell[t][c] = mine[32 * t + (half != 0 ? 1 + c : 0) * PT];
                }
            }
        }
        else
        {
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
            {
#pragma unroll
                for (int t = 0; t < TG; ++t)
                {
                    cell[t][KB + kb] = mine[32 * t + (KS + 2 * kb + half) * PT];
                }
#pragma unroll
                for (int t = 0; t < TG; ++t)
                {
                    cell[t][kb] = mine[32 * t + (2 * kb + half) * PT];
                }
            }
#pragma unroll
            for (int c = 0; c < G::NORM_TERMS; ++c)
            {
#pragma unroll
                for (int t = 0; t < TG; ++t)
                {
                    cell[t][2 * KB + c] = mine[32 * t + (2 * KS + (G::NORM_CELLS >= 2 ? 2 * c + half : c)) * PT];
                }
            }
        }
    };
    auto filter_values_and_cut = [&](const float* stage, vfloat16 (&w)[MT], int cut_base, auto mode_tag, auto sub_tag) __attribute__((always_inline)) {
        // (sub: which MT tiles of the stage; the cutting goes with the first ones)
        constexpr int SUB_PASS = decltype(sub_tag)::value;
        constexpr int MODE = SUB_PASS == 0 ? decltype(mode_tag)::value : 2;
        vfloat16 zero;
#pragma unroll
        for (int r = 0; r < 16; ++r)
        {
            zero[r] = 0.0F;
        }
        constexpr int TERMS = DP <= 8 ? 2 : 3 * KB + G::NORM_TERMS;
        constexpr int PAIRS_OF_VALUES = VPT / 2;
        constexpr int CHUNKS = MODE == 2 ? 0 : PAIRS_OF_VALUES + 1;
        static_assert(!EXACT || CHUNKS <= MT * TERMS, "a piece of the cutting per matrix instruction");
        float share = 0.0F;
        auto chunk = [&](auto c_tag) __attribute__((always_inline)) {
            constexpr int c = decltype(c_tag)::value;
            if constexpr (c < PAIRS_OF_VALUES)
            {
                // two values: pieces, share of the norm
                const vfloat2 pair{pre[2 * c], pre[2 * c + 1]};
                const u32 first = __builtin_bit_cast(u32, __builtin_convertvector(pair, vbf16x2));
                const vfloat2 rest{pair.x - __builtin_bit_cast(float, first << 16U),
                                   pair.y - __builtin_bit_cast(float, first & 0xFFFF0000U)};
                cut1[c] = first;
                cut2[c] = __builtin_bit_cast(u32, __builtin_convertvector(rest, vbf16x2));
                share = __builtin_fmaf(pair.x, pair.x, share);
                share = __builtin_fmaf(pair.y, pair.y, share);
            }
            else
            {
                if constexpr (PAIRED_SHARES)
                {
                    share += __builtin_bit_cast(float, lane_xor32<32>(__builtin_bit_cast(u32, share)));
                }
                const float lowered = __builtin_fmaf(-NORM_LOWER_DP, share, share);
                const vfloat2 whole{lowered, 0.0F};
                const u32 first = __builtin_bit_cast(u32, __builtin_convertvector(whole, vbf16x2)) & 0xFFFFU;
                const vfloat2 rest{lowered - __builtin_bit_cast(float, first << 16U), 0.0F};
                const u32 second = __builtin_bit_cast(u32, __builtin_convertvector(rest, vbf16x2)) & 0xFFFFU;
                cut_norm = cut_base + sp < n ? first | (second << 16U) : BF16_HUGE;
            }
        };
        if constexpr (NCELL > 12)
        {
            // (one tile whose cells do not fit the registers at once: they are read in pairs -- the
            // two cells of 16 dimensions that three matrix instructions take, then the two norm cells
            // of this half of the wave -- AHEAD pairs ahead of the instructions that take them)
            static_assert(MT == 1 && G::SUB == 1 && G::NORM_CELLS == 4);
            constexpr int AHEAD = 2;
            constexpr int PAIRS = KB + 1;
            const vuint4* const mine = reinterpret_cast<const vuint4*>(stage + DP * PT) + ql;
            vuint4 pair[AHEAD + 1][2];
            auto read_pair = [&](auto s_tag) __attribute__((always_inline)) {
                constexpr int at = decltype(s_tag)::value;
                if constexpr (at < KB)
                {
                    // piece 2, then piece 1, of dimensions 16 at ..
                    pair[at % (AHEAD + 1)][0] = mine[(KS + 2 * at + half) * PT];
                    pair[at % (AHEAD + 1)][1] = mine[(2 * at + half) * PT];
                }
                else if constexpr (at < PAIRS)
                {
                    pair[at % (AHEAD + 1)][0] = mine[(2 * KS + half) * PT];
                    pair[at % (AHEAD + 1)][1] = mine[(2 * KS + 2 + half) * PT];
                }
            };
            static_for<0, AHEAD>([&](auto s_tag) { read_pair(s_tag); });
            static_for<0, PAIRS>([&](auto s_tag) {
                constexpr int at = decltype(s_tag)::value;
                read_pair(std::integral_constant<int, at + AHEAD>{});
                constexpr int slot = at % (AHEAD + 1);
                if constexpr (at < KB)
                {
                    static_for<0, 3>([&](auto which_tag) {
                        constexpr int which = decltype(which_tag)::value;
                        constexpr int m = 3 * at + which;
                        w[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                            __builtin_bit_cast(vbf16x8, pair[slot][which == 0 ? 0 : 1]),
                            __builtin_bit_cast(vbf16x8, qs[which == 1 ? 1 : 0][at]), m == 0 ? zero : w[0], 0, 0, 0);
                        if constexpr (m < CHUNKS)
                        {
                            chunk(std::integral_constant<int, m>{});
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    });
                }
                else
                {
                    w[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(vbf16x8, pair[slot][0]),
                                                                   __builtin_bit_cast(vbf16x8, qs[2][0]), w[0], 0, 0, 0);
                    w[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(vbf16x8, pair[slot][1]),
                                                                   __builtin_bit_cast(vbf16x8, qs[2][0]), w[0], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
            });
        }
        else
        static_for<0, MT / TG>([&](auto g_tag) {
            constexpr int g = decltype(g_tag)::value;
            vuint4 cell[TG][NCELL];
            read_cells(stage, cell, SUB_PASS * MT + g * TG);
            __builtin_amdgcn_sched_barrier(0);
            static_for<0, TERMS>([&](auto j_tag) {
                constexpr int j = decltype(j_tag)::value;
                constexpr bool norm_term = DP > 8 && j >= 3 * KB;
                constexpr int kb = DP <= 8 || norm_term ? 0 : j / 3;
                constexpr int which = DP <= 8 ? j : j % 3;
                constexpr int a_at = DP <= 8 ? j : (norm_term ? 2 * KB + (j - 3 * KB) : (which == 0 ? KB + kb : kb));
                constexpr int b_piece = DP <= 8 ? j : (norm_term ? 2 : (which == 1 ? 1 : 0));
                constexpr int b_kb = kb;
                static_for<0, TG>([&](auto t_tag) {
                    constexpr int tt = decltype(t_tag)::value;
                    constexpr int t = g * TG + tt;
                    constexpr int m = (g * TERMS + j) * TG + tt; // number of this matrix instruction
                    w[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                        __builtin_bit_cast(vbf16x8, cell[tt][a_at]), __builtin_bit_cast(vbf16x8, qs[b_piece][b_kb]),
                        j == 0 ? zero : w[t], 0, 0, 0);
                    if constexpr (m < CHUNKS)
                    {
                        chunk(std::integral_constant<int, m>{});
                    }
                    __builtin_amdgcn_sched_barrier(0);
                });
            });
        });
    };
    // EXACT: the stage cut by filter_values_and_cut (fp32 rows from `pre`, cells from the pieces), or
    // the units of the image, into LDS; a handful of LDS writes.
    auto write_cut = [&](float* into, auto mode_tag) __attribute__((always_inline)) {
        constexpr int MODE = decltype(mode_tag)::value;
        if constexpr (MODE == 2)
        {
            static_for<0, IU>([&](auto j_tag) { deposit_image_unit(into, j_tag); });
        }
        else
        {
#pragma unroll
            for (int i = 0; i < VPT; ++i)
            {
                into[(sd0 + i) * PT + sp] = pre[i];
            }
            vuint4* const into_cells = reinterpret_cast<vuint4*>(into + DP * PT);
            constexpr int PIECE2 = DP <= 8 ? 1 : KS; // first cell of the second pieces
            if constexpr (VPT == 8)
            {
                into_cells[t] = vuint4{cut1[0], cut1[1], cut1[2], cut1[3]};
                into_cells[PIECE2 * PT + t] = vuint4{cut2[0], cut2[1], cut2[2], cut2[3]};
            }
            else
            {
                // half a cell per thread
                typedef u32 vuint2 __attribute__((ext_vector_type(2)));
                vuint2* const halves = reinterpret_cast<vuint2*>(into + DP * PT);
                const int h = sd0 / 4;
                halves[2 * sp + h] = vuint2{cut1[0], cut1[1]};
                halves[2 * (PIECE2 * PT + sp) + h] = vuint2{cut2[0], cut2[1]};
            }
            reinterpret_cast<u32*>(into_cells + (G::CELLS - G::NORM_CELLS + norm_slot / 4) * PT + sp)[norm_slot % 4] = cut_norm;
        }
    };
    // EXACT, second half of a stage.  First every tile is filtered without a branch: the smallest
    // filter value of every lane per tile and over the stage.  Only if some lane's is not above its
    // threshold are the lanes and rows of the tiles concerned collected, and the candidates of the
    // whole stage are worked through together.
    auto filter_and_append = [&](const vfloat16 (&w)[MT], const float* stage, int base) __attribute__((always_inline)) {
        float smallest[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t)
        {
            smallest[t] = smallest_of(w[t]);
        }
        float of_stage = smallest[0];
#pragma unroll
        for (int t = 1; t < MT; ++t)
        {
            of_stage = __builtin_elementwise_minimum(of_stage, smallest[t]);
        }
        // (negated compares: a NaN passes)
        const bool any = __builtin_amdgcn_ballot_w64(!(of_stage > thr)) != 0;
        BITSKNN_FT_LAP(3);
        if (any)
        {
            u32 part[MT];
            static_for<0, MT>([&](auto t_tag) {
                constexpr int t = decltype(t_tag)::value;
                part[t] = 0;
                if (__builtin_amdgcn_ballot_w64(!(smallest[t] > thr)) != 0)
                {
                    part[t] = bits_of(w[t]);
                }
            });
            u64 cand = part[0];
            if constexpr (MT >= 2)
            {
                cand |= static_cast<u64>(part[1]) << 16U;
            }
            if constexpr (MT == 4)
            {
                cand |= static_cast<u64>(part[2] | (part[3] << 16U)) << 32U;
            }
            exact_candidates(cand, stage, base);
        }
        BITSKNN_FT_LAP(4);
    };

    // all row tiles of a stage: distances, filter, append
    auto multiply = [&](const float* stage, int base) {
        if constexpr (EXACT)
        {
            vfloat16 w[MT];
            filter_values(stage, w);
            __builtin_amdgcn_sched_barrier(0);
            filter_and_append(w, stage, base);
        }
        else if constexpr (SPLIT)
        {
            constexpr int PAIRS = MT / 2;
            const vuint4* const cells = reinterpret_cast<const vuint4*>(stage);
            const float* const norm_row = stage + 3 * KS * PT * 4;
            static_for<0, PAIRS>([&](auto p_tag) {
                constexpr int p = decltype(p_tag)::value;
                // A operands of the two tiles: piece c of dimensions 16*kb + 8*half .. + 7
                vuint4 af[2][3][KB];
#pragma unroll
                for (int tile = 0; tile < 2; ++tile)
                {
#pragma unroll
                    for (int c = 0; c < 3; ++c)
                    {
#pragma unroll
                        for (int kb = 0; kb < KB; ++kb)
                        {
                            af[tile][c][kb] = cells[(c * KS + 2 * kb + half) * PT + p * 64 + tile * 32 + ql];
                        }
                    }
                }
                // the accumulators start from the norms of the lane's 16 points
                vfloat16 acc0;
                vfloat16 acc1;
                const float* norms = norm_row + p * 64 + 4 * half;
#pragma unroll
                for (int g = 0; g < 4; ++g)
                {
                    const vfloat4 x = *reinterpret_cast<const vfloat4*>(norms + 8 * g);
                    const vfloat4 y = *reinterpret_cast<const vfloat4*>(norms + 32 + 8 * g);
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                    {
                        acc0[4 * g + e] = x[e];
                        acc1[4 * g + e] = y[e];
                    }
                }
                // the six products of a step, smallest terms first
                constexpr int order[6][2] = {{2, 0}, {1, 1}, {0, 2}, {1, 0}, {0, 1}, {0, 0}};
                static_for<0, KB>([&](auto kb_tag) {
                    constexpr int kb = decltype(kb_tag)::value;
                    static_for<0, 6>([&](auto o_tag) {
                        constexpr int ca = order[decltype(o_tag)::value][0];
                        constexpr int cb = order[decltype(o_tag)::value][1];
                        acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                            __builtin_bit_cast(vbf16x8, af[0][ca][kb]), __builtin_bit_cast(vbf16x8, qs[cb][kb]),
                            acc0, 0, 0, 0);
                        acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                            __builtin_bit_cast(vbf16x8, af[1][ca][kb]), __builtin_bit_cast(vbf16x8, qs[cb][kb]),
                            acc1, 0, 0, 0);
                    });
                });
                filter_tile(acc0, base + p * 64);
                filter_tile(acc1, base + p * 64 + 32);
            });
            if constexpr (MT == 1)
            {
                // 64 dimensions: a stage is one tile
                vuint4 af[3][KB];
#pragma unroll
                for (int c = 0; c < 3; ++c)
                {
#pragma unroll
                    for (int kb = 0; kb < KB; ++kb)
                    {
                        af[c][kb] = cells[(c * KS + 2 * kb + half) * PT + ql];
                    }
                }
                vfloat16 acc;
#pragma unroll
                for (int g = 0; g < 4; ++g)
                {
                    const vfloat4 x = *reinterpret_cast<const vfloat4*>(norm_row + 4 * half + 8 * g);
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                    {
                        acc[4 * g + e] = x[e];
                    }
                }
                constexpr int order[6][2] = {{2, 0}, {1, 1}, {0, 2}, {1, 0}, {0, 1}, {0, 0}};
                static_for<0, KB>([&](auto kb_tag) {
                    constexpr int kb = decltype(kb_tag)::value;
                    static_for<0, 6>([&](auto o_tag) {
                        constexpr int ca = order[decltype(o_tag)::value][0];
                        constexpr int cb = order[decltype(o_tag)::value][1];
                        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                            __builtin_bit_cast(vbf16x8, af[ca][kb]), __builtin_bit_cast(vbf16x8, qs[cb][kb]), acc, 0,
                            0, 0);
                    });
                });
                filter_tile(acc, base);
            }
        }
        else if constexpr (MT >= 2)
        {
            // Two row tiles at a time: two independent accumulator chains keep the matrix core
            // issuing back to back.  The A operands of a pair sit in registers before its first
            // MFMA; those of the next pair are requested from LDS between the MFMAs of this one
            // (LDS instructions are overlapped with matrix instructions, vector-ALU ones are not).
            constexpr int PAIRS = MT / 2;
            float a[2][2][STEPS];
            // The reads of one tile are 2*PT floats apart, which a two-address LDS read with
            // offsets in units of 64 floats covers from one base register per tile; pairing the
            // two tiles of a step instead needs an address computation per step.
            const float* arow0 = stage + tile_at[0];
            const float* arow1 = stage + tile_at[1];
#pragma unroll
            for (int s = 0; s < STEPS; ++s)
            {
                a[0][0][s] = arow0[2 * s * PT];
            }
#pragma unroll
            for (int s = 0; s < STEPS; ++s)
            {
                a[0][1][s] = arow1[2 * s * PT];
            }
            // initial accumulators of a pair: zero, or the norms of the lane's 16 points
            vfloat16 init0;
            vfloat16 init1;
            auto request_init = [&](int pair) __attribute__((always_inline)) {
                if constexpr (NORM_IN_C)
                {
                    const float* norms = stage + DP * PT + pair * 64 + 4 * half;
#pragma unroll
                    for (int g = 0; g < 4; ++g)
                    {
                        const vfloat4 x = *reinterpret_cast<const vfloat4*>(norms + 8 * g);
                        const vfloat4 y = *reinterpret_cast<const vfloat4*>(norms + 32 + 8 * g);
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                        {
                            init0[4 * g + e] = x[e];
                            init1[4 * g + e] = y[e];
                        }
                    }
                }
                else
                {
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                    {
                        init0[r] = 0.0F;
                        init1[r] = 0.0F;
                    }
                }
            };
            request_init(0);
            __builtin_amdgcn_sched_barrier(0); // keep the reads above the chain
            static_for<0, PAIRS>([&](auto p_tag) {
                constexpr int p = decltype(p_tag)::value;
                constexpr int cur = p & 1;
                vfloat16 acc0 = init0;
                vfloat16 acc1 = init1;
                static_for<0, STEPS>([&](auto s_tag) {
                    constexpr int s = decltype(s_tag)::value;
                    if constexpr (p + 1 < PAIRS)
                    {
                        // steps (s, s+1) of the first tile in even steps, (s-1, s) of the second
                        // tile in odd ones
                        constexpr int next = 64 * (p + 1);
                        if constexpr (s % 2 == 0)
                        {
                            a[cur ^ 1][0][s] = arow0[2 * s * PT + next];
                            if constexpr (s + 1 < STEPS)
                            {
                                a[cur ^ 1][0][s + 1] = arow0[2 * (s + 1) * PT + next];
                            }
                            else
                            {
                                a[cur ^ 1][1][s] = arow1[2 * s * PT + next];
                            }
                        }
                        else
                        {
                            a[cur ^ 1][1][s - 1] = arow1[2 * (s - 1) * PT + next];
                            a[cur ^ 1][1][s] = arow1[2 * s * PT + next];
                        }
                    }
                    acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][0][s], qf[s], acc0, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][1][s], qf[s], acc1, 0, 0, 0);
                    if constexpr (NORM_IN_C && s == 0 && p + 1 < PAIRS)
                    {
                        request_init(p + 1); // the first step has taken this pair's
                    }
                    __builtin_amdgcn_sched_barrier(0);
                });
                filter_tile(acc0, base + p * 64);
                filter_tile(acc1, base + p * 64 + 32);
            });
        }
        else
        {
            vfloat16 acc0;
#pragma unroll
            for (int r = 0; r < 16; ++r)
            {
                acc0[r] = 0.0F;
            }
            const float* arow = stage + half * PT + ql;
#pragma unroll
            for (int s = 0; s < STEPS; ++s)
            {
                acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(arow[2 * s * PT], qf[s], acc0, 0, 0, 0);
            }
            if constexpr (VIA_F32)
            {
                // the tile's values are lower bounds (less the slack in thr): what is not above the
                // threshold is computed in the reference's arithmetic
                if (__builtin_amdgcn_ballot_w64(!(smallest_of(acc0) > thr)) != 0)
                {
                    exact_candidates(static_cast<u64>(bits_of(acc0)), stage, base);
                }
            }
            else
            {
                filter_tile(acc0, base);
            }
        }
    };

    // Stage s is multiplied while stage s+1 sits in registers and is written to the other LDS
    // buffer afterwards; stage s+2 is requested from memory right after that.  One barrier per
    // stage: it separates the last read of a buffer from its next fill and the fill from its
    // first read.  A wave that had to merge in stage s raises merge_wanted[s % 3]; the others look
    // at it before and after the barrier of that stage (the flag for stage s + 2 is cleared after the
    // barrier of stage s: its last readers passed it before that barrier, its next writers come
    // after the following one).
    auto merge_if_wanted = [&]() __attribute__((always_inline)) {
        if (!merged && __hip_atomic_load(merge_wanted + stage_slot, __ATOMIC_RELAXED,
                                         __HIP_MEMORY_SCOPE_WORKGROUP) != 0)
        {
            merge_event();
        }
    };
    if constexpr (!RING)
    {
        fetch(n_begin);
        // the query fragment and the first stage have arrived (nothing else is in flight yet)
        __builtin_amdgcn_s_waitcnt(0x0F70);
        deposit(stages, n_begin);
        if (n_begin + PT < n)
        {
            fetch(n_begin + PT);
        }
        __syncthreads();
        int parity = 0;
        for (int base = n_begin; base < n; base += PT)
        {
            merged = false;
            multiply(stages + parity * STAGE_FLOATS, base);
            parity ^= 1;
            if (base + PT < n)
            {
                deposit(stages + parity * STAGE_FLOATS, base + PT);
                if (base + 2 * PT < n)
                {
                    fetch(base + 2 * PT);
                }
            }
            if constexpr (JOIN_MERGES)
            {
                merge_if_wanted();
                __syncthreads();
                merge_if_wanted();
                if (t == 0)
                {
                    merge_wanted[(stage_slot + 2) % 3] = 0;
                }
                stage_slot = stage_slot == 2 ? 0 : stage_slot + 1;
            }
            else
            {
                __syncthreads();
            }
        }
    }
    else
    {
        // Ring of three stages.  A wave starts stage i when the stage is complete, writes its part of
        // stage i + 1 (requested from memory a stage earlier) and then multiplies stage i.  A wave
        // counts itself in at ready[slot] once its part of a stage is written (LDS executes the
        // instructions of a wave in order: the count follows the writes), and a stage is complete
        // when all waves have counted in: FQ_WAVES more per use of the slot.  There is no barrier: a
        // wave starts stage i + 1 as soon as every wave has started stage i, so one that appends or
        // merges holds up the others only when it falls a whole stage behind.  Stage i + 1 goes over
        // stage i - 2, which is safe once stage i is complete: every wave wrote its part of stage i
        // at the start of stage i - 1, after it had multiplied stage i - 2.
        // Every wave counts in for every stage whatever it finds in the tiles, and every wait is for
        // counts of an earlier point of the other waves' programs, so the counts are reached; the
        // bound on the polls only makes sure that a wave leaves the loop whatever happens.  A wave
        // whose wait ran out of polls goes on with a stage that may be incomplete, so it marks what
        // it reports at the end: NaN as the k-th distance of its queries and a count in *a.fault.
        static_assert(NB == 3);
        auto count_in = [&](int slot) __attribute__((always_inline)) {
            if (lane == 0)
            {
                __hip_atomic_fetch_add(ready + slot, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
        };
        auto wait_for = [&](int slot, int uses) __attribute__((always_inline)) {
            const int complete = FQ_WAVES * uses;
            int polls = a.poll_limit;
            while (__hip_atomic_load(ready + slot, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) < complete)
            {
                if (polls <= 0)
                {
                    gave_up = true;
                    break;
                }
                --polls;
                __builtin_amdgcn_s_sleep(1);
            }
        };
        if constexpr (!EXACT)
        {
            fetch(n_begin);
            // the query fragment and the first stage have arrived (nothing else is in flight yet)
            __builtin_amdgcn_s_waitcnt(0x0F70);
            deposit(stages, n_begin);
            count_in(0);
            if (n_begin + PT < n)
            {
                fetch(n_begin + PT);
            }
        }
        int slot = 0;  // of the stage being multiplied
        int round = 0; // how often that slot has been used before
        BITSKNN_FT_LAP(5);
        if constexpr (EXACT)
        {
            // The default arithmetic writes two stages ahead, at the end of an iteration.  Step k
            // writes stage k and counts at ready[k % 3]: steps 0 and 1 before the loop, step i + 2 at
            // the end of iteration i, which reads stage i.  Before it overwrites the slot of stage
            // i - 1 with stage i + 2, a wave waits until every wave has counted step i + 1, that is,
            // has finished iteration i - 1 (and written stage i + 1 at its end): the one wait of an
            // iteration also is what the next iteration's reads need.  So a wave may be a whole
            // iteration ahead of the slowest one of its workgroup -- the work on candidates differs
            // from wave to wave and stage to stage, and with less slack every wave pays for the
            // slowest one of every stage.  Every wave counts every step whatever its tiles hold,
            // and a wait is for counts that the other waves reach without waiting for this one.
            // The values of a stage are requested an iteration before they are cut (during the
            // matrix instructions) and written.  Past the last stage the waves write stages that
            // nobody reads (same waits, same counts).
            auto count_step = [&](int counter) __attribute__((always_inline)) {
                // (LDS executes the instructions of a wave in order: the count follows the writes
                // without a wait in between; the fence keeps the compiler from moving them)
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                if (lane == 0)
                {
                    __hip_atomic_fetch_add(ready + counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                }
            };
            auto pass = [&](auto mode_tag) __attribute__((always_inline)) {
                constexpr int MODE = decltype(mode_tag)::value; // 0: point matrices of 2 GiB and more,
                                                                // 1: buffer loads, 2: stages from an image
                auto request = [&](int base) __attribute__((always_inline)) {
                    if constexpr (MODE == 2)
                    {
                        fetch_image(base);
                    }
                    else if constexpr (MODE == 1)
                    {
                        // (buffer loads without a branch: beyond the matrix they read zero, and
                        // points from n on, whatever their values, carry the norm that only passes an
                        // infinite radius and are dropped by their labels)
                        const int stage_off = (base * a.sample_scale + a.sample_offset) * static_cast<int>(sizeof(float));
#pragma unroll
                        for (int i = 0; i < VPT; ++i)
                        {
                            pre[i] = __builtin_bit_cast(
                                float, __builtin_amdgcn_raw_buffer_load_b32(point_rsrc, load_off[i], stage_off, 0));
                        }
                    }
                    else
                    {
                        fetch(base < n ? base : n_begin);
                    }
                };
                auto write_whole = [&](float* into, int base) __attribute__((always_inline)) {
                    if constexpr (MODE == 2)
                    {
                        write_cut(into, mode_tag);
                    }
                    else
                    {
                        deposit(into, base);
                    }
                };
                request(n_begin);
                write_whole(stages, n_begin);
                count_step(0);
                request(n_begin + PT);
                wait_for(0, 1);
                write_whole(stages + STAGE_FLOATS, n_begin + PT);
                count_step(1);
                request(n_begin + 2 * PT);
                int reads = 0;   // slot of the stage being read (i % 3); its stage is complete
                int waits = 1;   // counter of step i + 1
                int writes = 2;  // slot of stage i + 2, counter of step i + 2
                int uses = 1;    // how often the counter `waits` has been used, this use included
                for (int base = n_begin; base < n; base += PT)
                {
                    BITSKNN_FT_LAP(0);
                    const float* const stage = stages + reads * STAGE_FLOATS;
                    static_for<0, G::SUB>([&](auto sub_tag) {
                        constexpr int sub = decltype(sub_tag)::value;
                        vfloat16 w[MT];
                        __builtin_amdgcn_sched_barrier(0);
                        filter_values_and_cut(stage, w, base + 2 * PT, mode_tag, sub_tag);
                        BITSKNN_FT_LAP(2);
                        filter_and_append(w, stage + 32 * MT * sub, base + 32 * MT * sub);
                    });
                    wait_for(waits, uses);
                    BITSKNN_FT_LAP(1);
                    write_cut(stages + writes * STAGE_FLOATS, mode_tag);
                    count_step(writes);
                    request(base + 3 * PT);
                    const int next = writes;
                    writes = reads;
                    reads = waits;
                    waits = next;
                    uses += waits == 0 ? 1 : 0;
                }
            };
            if (a.image != nullptr)
            {
                pass(std::integral_constant<int, 2>{});
            }
            else if (small_points)
            {
                pass(std::integral_constant<int, 1>{});
            }
            else
            {
                pass(std::integral_constant<int, 0>{});
            }
        }
        else
        for (int base = n_begin; base < n; base += PT)
        {
            wait_for(slot, round + 1);
            BITSKNN_FT_LAP(0);
#ifdef BITSKNN_FUSED_TIMING
            __builtin_amdgcn_s_waitcnt(0x0F70);
            BITSKNN_FT_LAP(1);
#endif
            if (base + PT < n)
            {
                const int next = slot + 1 == NB ? 0 : slot + 1;
                deposit(stages + next * STAGE_FLOATS, base + PT);
                count_in(next);
                if (base + 2 * PT < n)
                {
                    fetch(base + 2 * PT);
                }
            }
            BITSKNN_FT_LAP(2);
            multiply(stages + slot * STAGE_FLOATS, base);
            slot = slot + 1 == NB ? 0 : slot + 1;
            round += slot == 0 ? 1 : 0;
        }
    }

    // whatever is left in the buffers; also writes the lists of queries that never merged
    merge_event();
#ifdef BITSKNN_FUSED_TIMING
    BITSKNN_FT_LAP(6);
    if (lane == 0)
    {
        for (int i = 0; i < 8; ++i)
        {
            atomicAdd(a.timing + i, static_cast<unsigned long long>(ft_cycles[i]));
        }
    }
#endif
    // (the radius is the k-th distance of the finished list now if that is below the first radius)
    if (a.splits == 1 && first_radius < __builtin_inff() && !(radius < first_radius) && half == 0)
    {
        a.out_dist[static_cast<size_t>(my_q) * list_stride + K - 1] = __builtin_nanf("");
    }
    if constexpr (RING)
    {
        if (gave_up)
        {
            if (half == 0 && my_q < a.q)
            {
                a.out_dist[(static_cast<size_t>(my_q) * a.splits + blockIdx.y) * list_stride + K - 1] =
                    __builtin_nanf("");
            }
            if (lane == 0)
            {
                __hip_atomic_fetch_add(a.fault, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
}

template <int K, int DP, int ARITH, bool WIDE_OK, bool BIG_OK = false>
hipError_t launch_fused_as(const fused_args& a, hipStream_t stream)
{
    using G = fused_geometry<DP, ARITH, K, WIDE_OK, BIG_OK>;
    constexpr size_t lds_bytes = G::lds_bytes();
    if (lds_bytes > 48 * 1024)
    {
        const hipError_t status =
            hipFuncSetAttribute(reinterpret_cast<const void*>(&fused_kernel<K, DP, ARITH, WIDE_OK, BIG_OK>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
        if (status != hipSuccess)
        {
            return status;
        }
    }
    fused_args args = a;
    if (a.sample_scale > 1)
    {
        // every sample_scale-th stage, the one in the middle of its group
        constexpr int PT = G::PT;
        args.visit = a.n / (PT * a.sample_scale) * PT;
        args.sample_offset = a.sample_scale / 2 * PT;
        args.split_points = (args.visit + 255) / 256 * 256;
    }
    const unsigned grid = static_cast<unsigned>((a.q + G::QB - 1) / G::QB);
    hipLaunchKernelGGL((fused_kernel<K, DP, ARITH, WIDE_OK, BIG_OK>), dim3(grid, static_cast<unsigned>(a.splits)),
                       dim3(G::THREADS), lds_bytes, stream, args);
    return hipGetLastError();
}

// Launches over ranges of points take the 64-slot buffers where the geometry has them.  With one
// range of points the smaller stages cost more than the merges they save (65536 queries x 2^20
// points, k = 128: d = 8 19.5 ms with 64 slots, 17.3 ms with 32; d = 16 32.2 / 24.9 ms); over ranges
// the lists hardly converge and the merges weigh more (8192 queries x 2^17 points, d = 8, k = 256:
// 2.19 ms with 32 slots, 1.60 ms with 64).
template <int K, int DP, int ARITH>
hipError_t launch_fused(const fused_args& a, hipStream_t stream)
{
    if constexpr (fused_geometry<DP, ARITH, K, true>::WIDE)
    {
        if (a.splits > 1)
        {
            return launch_fused_as<K, DP, ARITH, true>(a, stream);
        }
    }
    // Workgroups of 256 queries where the caller of the launch chose them and the geometry has them
    // (no stage image: its stages are those of the workgroups of 128 queries)
    if constexpr (fused_geometry<DP, ARITH, K, false, true>::BIG)
    {
        if (a.workgroup > 0 && a.image == nullptr)
        {
            return launch_fused_as<K, DP, ARITH, false, true>(a, stream);
        }
    }
    return launch_fused_as<K, DP, ARITH, false>(a, stream);
}

} // namespace
} // namespace bitsknn

#endif // BITSKNN_CSRC_FUSED_KERNEL_HPP_
