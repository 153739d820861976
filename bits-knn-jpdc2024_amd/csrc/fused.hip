// C-ABI entry points of bits-fused: parameter validation, the choice between the fused kernel and
// its point-split form, and dispatch to the kernels instantiated per list length in fused_inst.hip.
#include <cstdlib>
#include <initializer_list>
#include <mutex>

#include "common.hpp"
#include "fused_args.hpp"

namespace bitsknn
{
namespace
{

// Scratch memory of bitsknn_fused_l2_topk_f32_static: the partial lists of the point ranges.
// Every GPU the library runs on holds its own copy of the array until the process ends.  In host
// code the array's name is only a handle for hipGetSymbolAddress; the device address it returns
// (one per device) is what kernels, copies and fills get.
constexpr size_t STATIC_SCRATCH_BYTES = 32ULL << 20;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

// Sticky fault word of the fused kernels (one copy per GPU, like `scratch`): the number of waits
// for a stage of the ring that ran out of polls since bitsknn_fused_status last looked.
static __device__ __align__(16) int fault_word[4];

#ifdef BITSKNN_FUSED_TIMING
static __device__ unsigned long long timing_words[8];
#endif

constexpr int MAX_DEVICES = 64;
// Default bound on the polls of one wait for a stage (each poll sleeps 64 cycles: about 0.1 s in
// all, many thousand times the longest merge a wave can be held up by).
constexpr int DEFAULT_POLL_LIMIT = 1 << 22;

struct device_symbols
{
    void* scratch = nullptr; // device addresses of this device's copies
    int* fault = nullptr;
};
std::mutex g_symbols_mutex;
device_symbols g_symbols[MAX_DEVICES];

// Device addresses of the current device's copies of `scratch` and `fault_word`, looked up on the
// first call per device.  Returns BITSKNN_OK or the status it has recorded with its message.
int symbols_of_current_device(device_symbols& out)
{
    int device = -1;
    BITSKNN_HIP_CHECK(hipGetDevice(&device));
    if (device < 0 || device >= MAX_DEVICES)
    {
        return fail(BITSKNN_ERR_INVALID, "bits-fused: device %d is not supported (at most %d)", device,
                    MAX_DEVICES);
    }
    const std::lock_guard<std::mutex> lock{g_symbols_mutex};
    device_symbols& mine = g_symbols[device];
    if (mine.fault == nullptr)
    {
        void* scratch_ptr = nullptr;
        void* fault_ptr = nullptr;
        BITSKNN_HIP_CHECK(hipGetSymbolAddress(&scratch_ptr, HIP_SYMBOL(scratch)));
        BITSKNN_HIP_CHECK(hipGetSymbolAddress(&fault_ptr, HIP_SYMBOL(fault_word)));
        mine.scratch = scratch_ptr;
        mine.fault = static_cast<int*>(fault_ptr);
    }
    out = mine;
    return BITSKNN_OK;
}

// Bound on the polls of a wait in the ring of stages: BITSKNN_FUSED_POLL_LIMIT in the environment
// (read once; 0 makes every wait that finds its stage incomplete give up at once, which is how the
// tests reach the failure path from the host), else DEFAULT_POLL_LIMIT.
int poll_limit()
{
    static const int limit = [] {
        const char* text = std::getenv("BITSKNN_FUSED_POLL_LIMIT");
        if (text != nullptr && *text != '\0')
        {
            char* end = nullptr;
            const long value = std::strtol(text, &end, 10);
            if (end != text && *end == '\0' && value >= 0 && value <= DEFAULT_POLL_LIMIT)
            {
                return static_cast<int>(value);
            }
        }
        return DEFAULT_POLL_LIMIT;
    }();
    return limit;
}

bool in_list(int v, std::initializer_list<int> values)
{
    for (const int x : values)
    {
        if (x == v)
        {
            return true;
        }
    }
    return false;
}

// Number of point ranges for a problem: enough workgroups for two per compute unit (one where a
// compute unit holds one: the exact arithmetic of 129 .. 256 dimensions, whose candidates start
// anew in every range -- 8192 queries x 2^17 points, d = 256, k = 32: 15.8 -> 13.1 ms with four
// ranges instead of eight), ranges of at least 4096 points and a multiple of 256, at most 64 ranges.
int choose_splits(int q, int n, int workgroups = 512)
{
    const int tiles = (q + FQ_QB - 1) / FQ_QB;
    int splits = 1;
    while (splits < 64 && tiles * splits < workgroups && n / (splits * 2) >= 4096)
    {
        splits *= 2;
    }
    return splits;
}

// The first radii of a launch come from a launch over a sample of the points, one stage in every
// `scale`: the value of rank r among a query's distances to the sample, r the smallest rank that
// at least r of the query's k nearest points fall into the sample (which is when fewer than k
// points lie below that value, and the query's workgroup has to repeat its pass) with a
// probability of at most 10^-10 for points in random order.  Returns 0 when the lists of the
// sample launch, which have min(k, 32) entries, do not reach that rank.
//
// One range of points (many queries): every 64th stage; lists of 128 and more only.  Measured on
// 65536 queries x 2^20 points: 51.6 -> 47.5 ms at k = 256 and 44.3 -> 43.7 ms at k = 128 in 32
// dimensions (26.1 -> 23.7 and 21.2 -> 20.6 ms in 8); up to k = 64 the launch over the sample costs
// more than the merges it saves.
//
// Several ranges (few queries): the list of a range hardly converges on its own (k (1 + ln(range / k))
// candidates per range and query), while hardly any point of a range lies below a radius taken
// from the whole point set (q = 8192, n = 2^17, d = 8: 2.66 -> 1.56 ms at k = 256, 1.31 -> 1.05 ms at
// k = 128, 0.88 -> 0.78 ms at k = 64; q = 1024, n = 2^20: 2.68 -> 1.04, 1.32 -> 0.88, 0.89 -> 0.76 ms).
// The sample launch runs on the few workgroups the queries give (it is not cut into ranges), so it
// takes about 2048 points whatever the point count (the constants below).
// The sweep over bitsknn_fused_tuning (bitsknn/tuning.py, fused_tuning.csv) is where these come
// from: with one range lists of 64 gain 1.5-4 % too (65536 queries x 2^20 points, d = 8: 9.63 ->
// 9.22 ms), and over ranges the sample wants about 2048 points whatever the point count (8192 queries
// x 2^17 points, k = 256: every 256th stage 2.05 ms, every 64th 1.38 ms; 1024 queries x 2^20 points
// are best served by every 256th).
constexpr int SAMPLE_SCALE = 64;
constexpr int SAMPLE_SCALE_RANGES_MIN = 64;
constexpr int SAMPLE_SCALE_RANGES_MAX = 256;
constexpr int SAMPLE_POINTS_RANGES = 2048;
constexpr int SAMPLE_MIN_POINTS = 1 << 17; // at least 8 (2 with ranges) sampled stages of any size
constexpr int SAMPLE_MIN_K = 64;
constexpr int SAMPLE_MIN_K_RANGES = 64; // (k <= 32: the three extra launches cost what the merges save)
// The stage image of the exact arithmetic is built, when the workspace has room for it, from this
// many queries on (its launch reads and writes the points once, about 0.1 ms for 2^20 points in 32
// dimensions; every workgroup of 128 queries saves the cutting of all its points) in up to this many
// dimensions (65536 queries x 2^20 points, k = 32: d = 8 7.4 -> 7.1 ms, d = 16 9.9 -> 9.6 ms, but
// d = 32 16.9 -> 17.3 ms and d = 64 33.2 -> 33.7 ms: the copy moves twice the bytes that the cutting
// reads, and there the vector instructions of the cutting hide behind the matrix instructions)
constexpr int IMAGE_MIN_QUERIES = 4096;
constexpr int IMAGE_MAX_DIM = 16;

int first_radius_rank(int k, int scale)
{
    const double p = 1.0 / scale;
    const int longest = k < 32 ? k : 32;
    // binomial(k, p) probabilities from the top down: the tail from r on
    double pmf[257];
    double value = 1.0;
    for (int i = 0; i < k; ++i)
    {
        value *= 1.0 - p;
    }
    for (int i = 0; i <= k; ++i)
    {
        pmf[i] = value;
        value *= static_cast<double>(k - i) / static_cast<double>(i + 1) * (p / (1.0 - p));
    }
    double tail = 0.0;
    int rank = k + 1;
    for (int i = k; i >= 1; --i)
    {
        tail += pmf[i];
        if (tail > 1e-10)
        {
            break;
        }
        rank = i;
    }
    return rank <= longest ? rank : 0;
}

hipError_t launch_for_k(int k, const fused_args& a, int arith, hipStream_t stream)
{
    switch (k)
    {
    case 4:
        return launch_fused_k_4(a, arith, stream);
    case 8:
        return launch_fused_k_8(a, arith, stream);
    case 16:
        return launch_fused_k_16(a, arith, stream);
    case 32:
        return launch_fused_k_32(a, arith, stream);
    case 64:
        return launch_fused_k_64(a, arith, stream);
    case 128:
        return launch_fused_k_128(a, arith, stream);
    default:
        return launch_fused_k_256(a, arith, stream);
    }
}

// bytes of the partial lists [q][splits][k]: distances, then labels
size_t partial_list_bytes(std::int32_t q, int splits, int k)
{
    return static_cast<size_t>(q) * static_cast<size_t>(splits) * static_cast<size_t>(k) * 8;
}

// use_workspace: the points may be cut into ranges whose partial lists go to `workspace`; a
// workspace too small for the ranges the problem would like gets as many as fit (a power of two,
// down to the single fused kernel that needs none).
int fused_impl(const float* queries_dim_major, const float* points_dim_major, int dim, std::int32_t q,
               std::int32_t n, float* out_dist, std::int32_t* out_label, int k, int query_reg,
               int db_reg, int dim_reg, int block_query_dim, int dim_mult, int arithmetic,
               void* workspace, size_t workspace_bytes, bool use_workspace, void* stream,
               const bitsknn_fused_tuning* tuning = nullptr)
{
    clear_error();
    if (tuning != nullptr)
    {
        if (tuning->ranges < 0 || tuning->ranges > 64)
        {
            return fail(BITSKNN_ERR_INVALID, "bitsknn_fused_tuning: ranges must be 0 (the library's choice) or 1 .. 64, got %d",
                        tuning->ranges);
        }
        if (tuning->first_radius < -1 || tuning->first_radius == 1 || tuning->first_radius > 4096)
        {
            return fail(BITSKNN_ERR_INVALID,
                        "bitsknn_fused_tuning: first_radius must be 0 (the library's choice), -1 (never) or 2 .. 4096 "
                        "(one stage in every so many), got %d",
                        tuning->first_radius);
        }
        if (tuning->image < -1 || tuning->image > 1)
        {
            return fail(BITSKNN_ERR_INVALID,
                        "bitsknn_fused_tuning: image must be 0 (the library's choice), -1 (never) or 1 (whenever the "
                        "workspace has room for it), got %d",
                        tuning->image);
        }
        if (tuning->workgroup != 0 && tuning->workgroup != 128 && tuning->workgroup != 256)
        {
            return fail(BITSKNN_ERR_INVALID,
                        "bitsknn_fused_tuning: workgroup must be 0 (the library's choice), 128 or 256 queries, got %d",
                        tuning->workgroup);
        }
        for (const std::int32_t word : tuning->reserved)
        {
            if (word != 0)
            {
                return fail(BITSKNN_ERR_INVALID, "bitsknn_fused_tuning: reserved words must be zero");
            }
        }
    }
    // the reference's nested dispatch, outermost first (fused_cache_knn.cu:72-144).  Its tuning
    // parameters describe a register tiling for the fp32 vector unit; they are validated like
    // there and have no effect on the tiling for the matrix cores, which is fixed by the
    // instruction shape (32 queries per wave) and by the dimension (points per stage)
    if (!in_list(query_reg, {2, 4, 8, 16}))
    {
        return fail(BITSKNN_ERR_UNSUPPORTED, "Unsupported queries_reg value: %d", query_reg);
    }
    if (!in_list(db_reg, {4, 8, 16}))
    {
        return fail(BITSKNN_ERR_UNSUPPORTED, "Unsupported db_reg value: %d", db_reg);
    }
    if (!in_list(dim_reg, {1, 2, 4}))
    {
        return fail(BITSKNN_ERR_UNSUPPORTED, "Unsupported dim_reg value: %d", dim_reg);
    }
    if (!in_list(block_query_dim, {1, 2, 4}))
    {
        return fail(BITSKNN_ERR_UNSUPPORTED, "Unsupported query_block_size value: %d", block_query_dim);
    }
    if (!in_list(dim_mult, {1, 2, 4}))
    {
        return fail(BITSKNN_ERR_UNSUPPORTED, "Unsupported dim_mult value: %d", dim_mult);
    }
    if (!in_list(k, {4, 8, 16, 32, 64, 128, 256}))
    {
        return fail(BITSKNN_ERR_UNSUPPORTED, "Unsupported k value: %d", k);
    }
    if (dim < dim_mult * dim_reg)
    {
        return fail(BITSKNN_ERR_UNSUPPORTED, "Dimension of vectors must not be lower than %d, but is %d",
                    dim_mult * dim_reg, dim);
    }
    if (arithmetic != BITSKNN_FUSED_FP32 && arithmetic != BITSKNN_FUSED_BF16X3 && arithmetic != BITSKNN_FUSED_EXACT)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_fused_l2_topk_f32: unknown arithmetic %d", arithmetic);
    }
    if (q <= 0)
    {
        return BITSKNN_OK;
    }
    if (n <= 0)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_fused_l2_topk_f32: no points");
    }
    if (queries_dim_major == nullptr || points_dim_major == nullptr || out_dist == nullptr ||
        out_label == nullptr)
    {
        return fail(BITSKNN_ERR_INVALID, "bitsknn_fused_l2_topk_f32: null pointer");
    }
    // (any int32 query count, as in the reference, fused_cache_kernel_structs.cuh:698-702: the
    // workgroups of 128 queries are the x dimension of the grid, which takes 2^31 - 1 of them)

    int splits = use_workspace && workspace != nullptr &&
                         reinterpret_cast<std::uintptr_t>(workspace) % 4 == 0
                     ? (tuning != nullptr && tuning->ranges > 0
                            ? tuning->ranges
                            : choose_splits(q, n, arithmetic == BITSKNN_FUSED_EXACT && dim > 128 && dim <= 256 ? 256 : 512))
                     : 1;
    // (ranges of at least one stage of the largest geometry)
    while (splits > 1 && n / splits < 256)
    {
        splits /= 2;
    }

    while (splits > 1 && partial_list_bytes(q, splits, k) > workspace_bytes)
    {
        splits /= 2;
    }
    const size_t pairs = static_cast<size_t>(q) * static_cast<size_t>(splits) * static_cast<size_t>(k);
    device_symbols symbols;
    const int looked_up = symbols_of_current_device(symbols);
    if (looked_up != BITSKNN_OK)
    {
        return looked_up;
    }
    fused_args a{queries_dim_major, points_dim_major, dim, q, n, out_dist, out_label, 1, 0, k, n, 1, 0, FUSED_PLAIN,
                 out_dist, k, symbols.fault, poll_limit()};
#ifdef BITSKNN_FUSED_TIMING
    {
        void* timing_ptr = nullptr;
        BITSKNN_HIP_CHECK(hipGetSymbolAddress(&timing_ptr, HIP_SYMBOL(timing_words)));
        a.timing = static_cast<unsigned long long*>(timing_ptr);
    }
#endif
    if (splits > 1)
    {
        // partial lists [q][splits][k] in the workspace: distances first, then labels
        a.out_dist = static_cast<float*>(workspace);
        a.out_label = reinterpret_cast<std::int32_t*>(a.out_dist + pairs);
        a.splits = splits;
    }
    a.split_points = ((n + splits - 1) / splits + 255) / 256 * 256;
    a.image = nullptr;
    a.image_bytes = 0;
    // Workgroups of 256 queries (eight waves sharing stages of twice the points: half the staging,
    // LDS writes and hand-overs per pair) where the kernel has them and they fill the chip: one per
    // compute unit, ranges of points included.  65536 queries x 2^20 points, k = 32: d = 8 7.65 ->
    // 6.40 ms, d = 16 10.1 -> 8.86 ms, d = 32 16.8 -> 14.3 ms (the stage image, which only the
    // workgroups of 128 queries take, gives 7.10 / 9.82 / 17.2 ms).
    // Every list length has the shape (its LDS holds the ring of stages for all of them), but long
    // lists gain from it only where merges are not what the time goes into -- one range of points,
    // and the longer the list the more dimensions (65536 queries x 2^20 points, 128 -> 256 queries per
    // workgroup: k = 64 d = 16 / 32 / 64 13.4 -> 10.8, 23.0 -> 17.1, 46.1 -> 28.6 ms; k = 128 d = 16 14.5 ->
    // 15.4 but d = 32 / 64 25.0 -> 20.7, 51.4 -> 33.1 ms; k = 256 d = 32 28.4 -> 33.7 but d = 64 58.8 ->
    // 47.4 ms; over ranges 8192 x 2^17, d = 32, k = 128: 1.23 -> 1.83 ms): the waves of the smaller
    // workgroups merge long lists together at a barrier, these each on its own.
    // (65 .. 128 dimensions have the exact arithmetic in this shape only)
    const bool has_big = arithmetic == BITSKNN_FUSED_EXACT && dim <= 128;
    const bool only_big = has_big && dim > 64;
    // (Over ranges, lists of 64 gain above 32 dimensions -- 4096 x 2^20, d = 64: 4.7 -> 3.4 ms,
    // 8192 x 2^17: 1.78 -> 1.60 ms -- and lists of 128 where a range has at least 2^18 points: 16384 x
    // 2^20, d = 64: 16.1 -> 13.1 ms, but 8192 x 2^17: 2.05 -> 2.53 ms.)
    const bool long_ranges = splits == 1 || n / splits >= (1 << 18);
    const bool big_pays = k <= 32 || (dim <= 8 && k <= 64) || (k == 64 && (splits == 1 || dim > 32)) ||
                          (k == 128 && dim > 16 && long_ranges) || (k == 256 && dim > 32 && splits == 1);
    const long long big_workgroups = (static_cast<long long>(q) + 255) / 256 * splits;
    // (every compute unit runs one of them at a time: they are taken where their last round leaves
    // at most an eighth of the units idle -- 224 .. 256, 448 .. 512, ... -- since workgroups of
    // 128 queries, two to a unit, end a ragged last round sooner: 49152 queries x 2^20 points over
    // two ranges, d = 16: 9.6 ms against 10.2 ms)
    const long long big_rounds = (big_workgroups + 255) / 256;
    const bool big_fills = 8 * big_workgroups >= 7 * 256 * big_rounds;
    const bool big =
        has_big && (only_big || (tuning != nullptr && tuning->workgroup != 0 ? tuning->workgroup == 256
                                                                             : big_fills && big_pays));
    a.workgroup = big ? 1 : 0;

    auto* hip_stream = static_cast<hipStream_t>(stream);
    const int split = arithmetic == BITSKNN_FUSED_BF16X3 ? FUSED_ARITH_BF16X3
                      : arithmetic == BITSKNN_FUSED_EXACT ? FUSED_ARITH_EXACT
                                                          : FUSED_ARITH_MFMA_F32;
    // one bits pass over the splits*k candidates of every query, labels carried along
    auto reduce_ranges = [&]() -> int {
        const size_t cols = static_cast<size_t>(splits) * static_cast<size_t>(k);
        return bitsknn_topk_bits_f32(a.out_dist, cols, a.out_label, cols, nullptr, static_cast<size_t>(q), cols,
                                     out_dist, out_label, static_cast<size_t>(k), static_cast<std::uint32_t>(k),
                                     128, 4, 0, stream);
    };
    hipError_t status = hipSuccess;
    // The stage image: with room for it in the workspace behind the partial lists, the points are
    // cut into the stages of the exact arithmetic once, by a launch of their own, instead of by
    // every workgroup of the fused kernel again.  That pays from a few thousand queries on.
    if (split == FUSED_ARITH_EXACT && use_workspace && workspace != nullptr && dim <= 64 && !big &&
        (tuning == nullptr || tuning->image >= 0))
    {
        const size_t image_bytes = fused_image_bytes(dim, n);
        const size_t lists = splits > 1 ? partial_list_bytes(q, splits, k) : 0;
        const size_t offset = (lists + 255) / 256 * 256;
        const bool wanted =
            (tuning != nullptr && tuning->image == 1) || (q >= IMAGE_MIN_QUERIES && dim <= IMAGE_MAX_DIM);
        if (wanted && image_bytes > 0 && image_bytes < (1ULL << 31) && offset + image_bytes <= workspace_bytes &&
            reinterpret_cast<std::uintptr_t>(workspace) % 16 == 0)
        {
            void* const image = static_cast<char*>(workspace) + offset;
            status = launch_fused_image(points_dim_major, dim, n, image, hip_stream);
            BITSKNN_HIP_CHECK(status);
            a.image = image;
            a.image_bytes = static_cast<int>(image_bytes);
        }
    }
    int scale = SAMPLE_SCALE;
    if (splits > 1)
    {
        scale = n / SAMPLE_POINTS_RANGES;
        scale = scale < SAMPLE_SCALE_RANGES_MIN ? SAMPLE_SCALE_RANGES_MIN
                                                : (scale > SAMPLE_SCALE_RANGES_MAX ? SAMPLE_SCALE_RANGES_MAX : scale);
    }
    // (more than 256 dimensions: the plain kernel of any_dim.hip, whatever the arithmetic asked for;
    // it takes the ranges of points but neither first radii nor the other launch parameters)
    const bool any_dim = dim > 256;
    bool sample = n >= SAMPLE_MIN_POINTS && k >= (splits == 1 ? SAMPLE_MIN_K : SAMPLE_MIN_K_RANGES);
    if (tuning != nullptr && tuning->first_radius != 0)
    {
        // the caller's choice, as far as the sample has at least two stages of any geometry
        sample = tuning->first_radius > 0 && n / tuning->first_radius >= 512;
        scale = sample ? tuning->first_radius : scale;
    }
    sample = sample && !any_dim;
    const int rank = sample ? first_radius_rank(k, scale) : 0;
    if (rank > 0)
    {
        // lists of min(k, 32) nearest sample points into the first entries of the caller's output
        // rows, one range; the launch below takes its first radii from them, and they are
        // overwritten by its lists (one range) or by the reduced lists (several)
        fused_args sample = a;
        sample.out_dist = out_dist;
        sample.out_label = out_label;
        sample.splits = 1;
        sample.sample_scale = scale;
        status = launch_for_k(k < 32 ? k : 32, sample, split, hip_stream);
        BITSKNN_HIP_CHECK(status);
        a.first_radius = FUSED_FIRST_RADIUS_FROM + rank - 1;
    }
    status = any_dim ? launch_fused_any_dim(a, k, hip_stream) : launch_for_k(k, a, split, hip_stream);
    BITSKNN_HIP_CHECK(status);
    if (splits > 1)
    {
        const int reduced = reduce_ranges();
        if (reduced != BITSKNN_OK)
        {
            return reduced;
        }
    }
    if (rank > 0)
    {
        // the workgroups with a query whose first radius proved too low repeat their pass from
        // +inf (all ranges of such a query); the others leave at once
        a.first_radius = FUSED_REPEAT_MARKED;
        status = launch_for_k(k, a, split, hip_stream);
        BITSKNN_HIP_CHECK(status);
        if (splits > 1)
        {
            return reduce_ranges();
        }
    }
    return BITSKNN_OK;
}

} // namespace
} // namespace bitsknn

extern "C" int bitsknn_fused_l2_topk_f32(const float* queries_dim_major,
                                         const float* points_dim_major, int dim, int32_t q,
                                         int32_t n, float* out_dist, int32_t* out_label, int k,
                                         int query_reg, int db_reg, int dim_reg, int block_query_dim,
                                         int dim_mult, void* stream)
{
    return bitsknn::fused_impl(queries_dim_major, points_dim_major, dim, q, n, out_dist, out_label, k,
                               query_reg, db_reg, dim_reg, block_query_dim, dim_mult, BITSKNN_FUSED_EXACT,
                               nullptr, 0, false, stream);
}

extern "C" size_t bitsknn_fused_image_bytes(int dim, int32_t n)
{
    const size_t bytes = bitsknn::fused_image_bytes(dim, n);
    return bytes < (1ULL << 31) ? bytes : 0;
}

extern "C" size_t bitsknn_fused_workspace_bytes(int32_t q, int32_t n, int k)
{
    if (q <= 0 || n <= 0 || k <= 0)
    {
        return 0;
    }
    const int splits = bitsknn::choose_splits(q, n);
    return splits > 1 ? bitsknn::partial_list_bytes(q, splits, k) : 0;
}

extern "C" int bitsknn_fused_l2_topk_f32_ws(const float* queries_dim_major,
                                            const float* points_dim_major, int dim, int32_t q,
                                            int32_t n, float* out_dist, int32_t* out_label, int k,
                                            int query_reg, int db_reg, int dim_reg,
                                            int block_query_dim, int dim_mult, void* workspace,
                                            size_t workspace_bytes, void* stream)
{
    return bitsknn::fused_impl(queries_dim_major, points_dim_major, dim, q, n, out_dist, out_label, k,
                               query_reg, db_reg, dim_reg, block_query_dim, dim_mult, BITSKNN_FUSED_EXACT,
                               workspace, workspace_bytes, true, stream);
}

extern "C" int bitsknn_fused_l2_topk_f32_ex(const float* queries_dim_major,
                                            const float* points_dim_major, int dim, int32_t q,
                                            int32_t n, float* out_dist, int32_t* out_label, int k,
                                            int query_reg, int db_reg, int dim_reg,
                                            int block_query_dim, int dim_mult, int arithmetic,
                                            void* workspace, size_t workspace_bytes, void* stream)
{
    return bitsknn::fused_impl(queries_dim_major, points_dim_major, dim, q, n, out_dist, out_label, k,
                               query_reg, db_reg, dim_reg, block_query_dim, dim_mult, arithmetic, workspace,
                               workspace_bytes, workspace != nullptr, stream);
}

extern "C" int bitsknn_fused_l2_topk_f32_tuned(const float* queries_dim_major,
                                               const float* points_dim_major, int dim, int32_t q,
                                               int32_t n, float* out_dist, int32_t* out_label, int k,
                                               int arithmetic, const bitsknn_fused_tuning* tuning,
                                               void* workspace, size_t workspace_bytes, void* stream)
{
    // (the reference's five parameters at the values of its fixed choice: they only have to be valid)
    return bitsknn::fused_impl(queries_dim_major, points_dim_major, dim, q, n, out_dist, out_label, k, 2, 4, 1, 1,
                               1, arithmetic, workspace, workspace_bytes, workspace != nullptr, stream, tuning);
}

extern "C" size_t bitsknn_fused_static_scratch_bytes(void) { return bitsknn::STATIC_SCRATCH_BYTES; }

extern "C" int bitsknn_fused_l2_topk_f32_static(const float* queries_dim_major,
                                                const float* points_dim_major, int dim, int32_t q,
                                                int32_t n, float* out_dist, int32_t* out_label, int k,
                                                int query_reg, int db_reg, int dim_reg,
                                                int block_query_dim, int dim_mult, void* stream)
{
    using namespace bitsknn;
    // parameter errors first, with the messages of the other entry points (no queries: validation only)
    const int valid = fused_impl(queries_dim_major, points_dim_major, dim, 0, n, out_dist, out_label, k,
                                 query_reg, db_reg, dim_reg, block_query_dim, dim_mult, BITSKNN_FUSED_EXACT,
                                 nullptr, 0, false, stream);
    if (valid != BITSKNN_OK)
    {
        return valid;
    }
    const size_t need = bitsknn_fused_workspace_bytes(q, n, k);
    if (need > STATIC_SCRATCH_BYTES)
    {
        return fail(BITSKNN_ERR_INVALID,
                    "bitsknn_fused_l2_topk_f32_static: the partial lists of this problem take %zu bytes, the "
                    "library's own scratch memory holds %zu (use bitsknn_fused_l2_topk_f32_ws)",
                    need, STATIC_SCRATCH_BYTES);
    }
    void* workspace = nullptr;
    if (need != 0 && q > 0)
    {
        device_symbols symbols;
        const int looked_up = symbols_of_current_device(symbols);
        if (looked_up != BITSKNN_OK)
        {
            return looked_up;
        }
        workspace = symbols.scratch;
    }
    // The kernels write every entry of the partial lists they read back (ranges without points
    // included), so nothing in the scratch memory has to be cleared between calls.
    return fused_impl(queries_dim_major, points_dim_major, dim, q, n, out_dist, out_label, k, query_reg,
                      db_reg, dim_reg, block_query_dim, dim_mult, BITSKNN_FUSED_EXACT, workspace,
                      workspace != nullptr ? STATIC_SCRATCH_BYTES : 0, workspace != nullptr, stream);
}

extern "C" int bitsknn_fused_status(void* stream)
{
    using namespace bitsknn;
    clear_error();
    device_symbols symbols;
    const int looked_up = symbols_of_current_device(symbols);
    if (looked_up != BITSKNN_OK)
    {
        return looked_up;
    }
    auto* hip_stream = static_cast<hipStream_t>(stream);
    int gave_up = 0;
    BITSKNN_HIP_CHECK(hipMemcpyAsync(&gave_up, symbols.fault, sizeof(int), hipMemcpyDeviceToHost, hip_stream));
    BITSKNN_HIP_CHECK(hipStreamSynchronize(hip_stream));
    if (gave_up == 0)
    {
        return BITSKNN_OK;
    }
    static const int zero = 0;
    BITSKNN_HIP_CHECK(hipMemcpyAsync(symbols.fault, &zero, sizeof(int), hipMemcpyHostToDevice, hip_stream));
    BITSKNN_HIP_CHECK(hipStreamSynchronize(hip_stream));
    return fail(BITSKNN_ERR_INTERNAL,
                "bits-fused: %d waits for a stage ran out of polls; the lists of the queries concerned end "
                "in NaN and the results of the calls since the last check must be discarded",
                gave_up);
}

#ifdef BITSKNN_FUSED_TIMING
// instrumented build only: synchronises, copies the eight cycle sums out and clears them
extern "C" int bitsknn_fused_timing(unsigned long long* out8, void* stream)
{
    using namespace bitsknn;
    auto* hip_stream = static_cast<hipStream_t>(stream);
    void* timing_ptr = nullptr;
    BITSKNN_HIP_CHECK(hipGetSymbolAddress(&timing_ptr, HIP_SYMBOL(timing_words)));
    BITSKNN_HIP_CHECK(hipStreamSynchronize(hip_stream));
    BITSKNN_HIP_CHECK(hipMemcpy(out8, timing_ptr, 8 * sizeof(unsigned long long), hipMemcpyDeviceToHost));
    static const unsigned long long zeros[8] = {};
    BITSKNN_HIP_CHECK(hipMemcpy(timing_ptr, zeros, sizeof(zeros), hipMemcpyHostToDevice));
    return BITSKNN_OK;
}
#endif
