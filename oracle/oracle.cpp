/*
 * CPU oracle for the k-NN hot path -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Only the test-suite, the smoke test and the CPU-baseline leg of the benchmark may load
 * this library; it is the checker, never the thing that is measured as the product or
 * shipped.  Paths cited below are relative to the reference tree.
 *
 * What pins each function (so that a plausible mistake fails a test):
 *   oracle_engine_init / oracle_uniform_fill / oracle_normal_fill
 *       - bit-compared with the reference's own generator headers compiled unmodified
 *         (oracle/_ref, built from include/bits/generator/ *.hpp);
 *       - end to end by the reference-held checksums (data/ *.err): a wrong stream cannot
 *         reproduce them.
 *   oracle_preprocess_ordering, oracle_parse_number, oracle_parse_dim3
 *       - bit-compared with the reference headers in oracle/_ref; closed-form checksums
 *         k(k-1)/2 (ascending) and sum_{i=n-k}^{n-1} i (descending) held in data/buffer-*.err.
 *   oracle_dist_l2
 *       - reference-held checksums of the k-selection runs (d = 1) and fused runs (d = 4, 8, 16);
 *         fp64 triple loop as the mathematical truth.
 *   oracle_dist_partial_l2
 *       - identity ||p||^2 - 2 q.p = ||q-p||^2 - ||q||^2 against the fp64 truth; neighbour
 *         sets against the fused-run checksums.
 *   oracle_topk
 *       - brute force (full stable sort by (value, label)) on small inputs; invariants; all
 *         unanimous reference-held checksums.
 *   oracle_topk_serial, oracle_topk_parallel
 *       - same multiset of values as oracle_topk on every input, same labels on tie-free
 *         inputs.
 *   oracle_verify
 *       - hand-built cases: identical, boundary-tie permutation (accepted), real mismatch
 *         (rejected).  No reference-held vector exists for it ("parity unpinned" beyond those
 *         hand cases: the reference ignores verify()'s result, src/main.cpp:420-436).
 */
#include "oracle.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <string>
#include <utility>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

namespace
{

// std::default_random_engine of libstdc++ is minstd_rand0: x <- 16807 x mod (2^31 - 1).
constexpr uint64_t LCG_A = 16807;
constexpr uint64_t LCG_M = 2147483647;

inline uint32_t lcg_next(uint32_t x) { return static_cast<uint32_t>((LCG_A * x) % LCG_M); }

uint64_t mulmod(uint64_t a, uint64_t b) { return (a * b) % LCG_M; } // operands < 2^31

uint64_t powmod(uint64_t base, uint64_t exp)
{
    uint64_t result = 1;
    base %= LCG_M;
    while (exp != 0)
    {
        if ((exp & 1U) != 0)
        {
            result = mulmod(result, base);
        }
        base = mulmod(base, base);
        exp >>= 1U;
    }
    return result;
}

// std::generate_canonical<float, 24>(minstd_rand0): one draw, (x - min) / (max - min + 1) in
// float where the divisor 2147483646 rounds to 2^31, clamped below 1.
inline float canonical(uint32_t x)
{
    const float sum = static_cast<float>(x - 1U);
    const float range = 2147483648.0F;
    float ret = sum / range;
    if (ret >= 1.0F)
    {
        ret = std::nextafter(1.0F, 0.0F);
    }
    return ret;
}

struct pair_t
{
    float distance;
    int32_t index;
};

inline bool pair_less(const pair_t& a, const pair_t& b)
{
    return a.distance < b.distance || (a.distance == b.distance && a.index < b.index);
}

// floating point comparison of src/verify.cpp:17-35
bool approx_equal(float a, float b, float epsilon)
{
    const float abs_a = std::abs(a);
    const float abs_b = std::abs(b);
    const float diff = std::abs(a - b);
    if (a == b)
    {
        return true;
    }
    if (a == 0 || b == 0 || (abs_a + abs_b < std::numeric_limits<float>::min()))
    {
        return diff < (epsilon * std::numeric_limits<float>::min());
    }
    return diff / std::min<float>(abs_a + abs_b, std::numeric_limits<float>::max()) < epsilon;
}

// src/verify.cpp:37-51
void normalize(std::vector<pair_t>& data)
{
    const float eps = 1e-3F;
    for (int32_t i = 1; i < static_cast<int32_t>(data.size()); ++i)
    {
        int32_t j = i;
        while (j > 0 && approx_equal(data[j].distance, data[j - 1].distance, eps) &&
               data[j].index > data[j - 1].index)
        {
            std::swap(data[j], data[j - 1]);
            --j;
        }
    }
}

// src/verify.cpp:53-74
bool same_distance(const pair_t* begin, const pair_t* end)
{
    const float eps = 1e-3F;
    if (begin == end)
    {
        return false;
    }
    const pair_t* prev = begin;
    for (const pair_t* it = begin + 1; it != end; ++it)
    {
        if (!approx_equal(prev->distance, it->distance, eps))
        {
            return false;
        }
        prev = it;
    }
    return true;
}

} // namespace

extern "C" {

uint32_t oracle_engine_init(uint64_t seed)
{
    // linear_congruential_engine::seed: x = seed mod m, and 1 if that is 0 (increment is 0)
    uint64_t x = seed % LCG_M;
    if (x == 0)
    {
        x = 1;
    }
    return oracle_engine_skip(static_cast<uint32_t>(x), 1U << 12U);
}

uint32_t oracle_engine_skip(uint32_t state, uint64_t steps)
{
    return static_cast<uint32_t>(mulmod(state, powmod(LCG_A, steps)));
}

uint32_t oracle_uniform_fill(uint32_t state, float lo, float hi, float* out, size_t count)
{
    const float width = hi - lo;
    const long long total = static_cast<long long>(count);
    const long long block = 1LL << 16;
    const long long blocks = (total + block - 1) / block;
#pragma omp parallel for schedule(static) if (total > (1LL << 20))
    for (long long b = 0; b < blocks; ++b)
    {
        const long long begin = b * block;
        const long long end = std::min(total, begin + block);
        uint32_t x = oracle_engine_skip(state, static_cast<uint64_t>(begin));
        for (long long i = begin; i < end; ++i)
        {
            x = lcg_next(x);
            // uniform_real_distribution: canonical * (b - a) + a, two roundings
            const float scaled = canonical(x) * width;
            out[i] = scaled + lo;
        }
    }
    return oracle_engine_skip(state, count);
}

uint32_t oracle_normal_fill(uint32_t state, float mean, float stddev, float* out, size_t count)
{
    uint32_t x = state;
    bool saved_available = false;
    float saved = 0;
    for (size_t i = 0; i < count; ++i)
    {
        float ret = 0;
        if (saved_available)
        {
            saved_available = false;
            ret = saved;
        }
        else
        {
            float u = 0;
            float v = 0;
            float r2 = 0;
            do
            {
                x = lcg_next(x);
                u = static_cast<float>(2.0F * canonical(x) - 1.0);
                x = lcg_next(x);
                v = static_cast<float>(2.0F * canonical(x) - 1.0);
                const float uu = u * u;
                const float vv = v * v;
                r2 = uu + vv;
            } while (r2 > 1.0 || r2 == 0.0);
            const float mult = std::sqrt(-2 * std::log(r2) / r2);
            saved = u * mult;
            saved_available = true;
            ret = v * mult;
        }
        const float scaled = ret * stddev;
        out[i] = scaled + mean;
    }
    return x;
}

void oracle_preprocess_ordering(float* data, size_t data_floats, float* query, size_t query_floats,
                                int descending)
{
    std::fill(query, query + query_floats, 0.0F);
    if (descending != 0)
    {
        std::sort(data, data + data_floats, [](float a, float b) { return a > b; });
    }
    else
    {
        std::sort(data, data + data_floats, [](float a, float b) { return a < b; });
    }
}

uint64_t oracle_parse_number(const char* text)
{
    std::string number{text};
    if (number.empty())
    {
        return 0;
    }
    uint64_t multiplier = 1;
    const char last = number.back();
    if (last == 'k' || last == 'K')
    {
        multiplier = 1ULL << 10U;
        number.pop_back();
    }
    else if (last == 'm' || last == 'M')
    {
        multiplier = 1ULL << 20U;
        number.pop_back();
    }
    else if (last == 'g' || last == 'G')
    {
        multiplier = 1ULL << 30U;
        number.pop_back();
    }
    return static_cast<uint64_t>(std::atol(number.c_str())) * multiplier;
}

void oracle_parse_dim3(const char* text, uint64_t out[3])
{
    out[0] = out[1] = out[2] = 1;
    std::vector<std::string> parts(1);
    for (const char* c = text; *c != '\0'; ++c)
    {
        if (*c == ',')
        {
            parts.emplace_back();
        }
        else
        {
            parts.back().push_back(*c);
        }
    }
    for (size_t i = 0; i < std::min<size_t>(3, parts.size()); ++i)
    {
        out[i] = oracle_parse_number(parts[i].c_str());
    }
}

void oracle_dist_l2(const float* queries, const float* points, size_t q, size_t n, size_t d,
                    float* out, size_t out_stride)
{
#pragma omp parallel for schedule(static)
    for (long long i = 0; i < static_cast<long long>(q); ++i)
    {
        const float* qv = queries + static_cast<size_t>(i) * d;
        for (size_t j = 0; j < n; ++j)
        {
            const float* pv = points + j * d;
            float acc = 0;
            for (size_t t = 0; t < d; ++t)
            {
                const float diff = qv[t] - pv[t];
                acc = std::fmaf(diff, diff, acc);
            }
            out[static_cast<size_t>(i) * out_stride + j] = acc;
        }
    }
}

void oracle_dist_partial_l2(const float* queries, const float* points, size_t q, size_t n, size_t d,
                            float* out, size_t out_stride)
{
#pragma omp parallel for schedule(static)
    for (long long i = 0; i < static_cast<long long>(q); ++i)
    {
        const float* qv = queries + static_cast<size_t>(i) * d;
        for (size_t j = 0; j < n; ++j)
        {
            const float* pv = points + j * d;
            float norm = 0;
            float dot = 0;
            for (size_t t = 0; t < d; ++t)
            {
                norm = std::fmaf(pv[t], pv[t], norm);
                dot = std::fmaf(qv[t], pv[t], dot);
            }
            // norm - 2*dot: 2*dot is exact, so one rounding either way
            out[static_cast<size_t>(i) * out_stride + j] = std::fmaf(-2.0F, dot, norm);
        }
    }
}

void oracle_dist_f64(const float* queries, const float* points, size_t q, size_t n, size_t d,
                     int partial, double* out, size_t out_stride)
{
#pragma omp parallel for schedule(static)
    for (long long i = 0; i < static_cast<long long>(q); ++i)
    {
        const float* qv = queries + static_cast<size_t>(i) * d;
        for (size_t j = 0; j < n; ++j)
        {
            const float* pv = points + j * d;
            double acc = 0;
            for (size_t t = 0; t < d; ++t)
            {
                const double a = qv[t];
                const double b = pv[t];
                acc += partial != 0 ? (b * b - 2.0 * a * b) : (a - b) * (a - b);
            }
            out[static_cast<size_t>(i) * out_stride + j] = acc;
        }
    }
}

void oracle_topk(const float* in, size_t in_stride, const int32_t* labels, size_t label_stride,
                 const int32_t* label_offsets, size_t rows, size_t cols, size_t k,
                 float* out_dist, int32_t* out_label, size_t out_stride)
{
#pragma omp parallel for schedule(dynamic)
    for (long long r = 0; r < static_cast<long long>(rows); ++r)
    {
        const float* row = in + static_cast<size_t>(r) * in_stride;
        const size_t take = std::min(k, cols);
        std::vector<pair_t> cand;
        auto label_of = [&](size_t c) {
            int32_t label = labels != nullptr ? labels[static_cast<size_t>(r) * label_stride + c]
                                              : static_cast<int32_t>(c);
            if (label_offsets != nullptr)
            {
                label = static_cast<int32_t>(static_cast<uint32_t>(label) +
                                             static_cast<uint32_t>(label_offsets[r]));
            }
            return label;
        };
        if (take > 0)
        {
            // value of the take-th smallest element, then every element not above it
            std::vector<float> copy(row, row + cols);
            std::nth_element(copy.begin(), copy.begin() + (take - 1), copy.end());
            const float threshold = copy[take - 1];
            for (size_t c = 0; c < cols; ++c)
            {
                if (row[c] <= threshold)
                {
                    cand.push_back(pair_t{row[c], label_of(c)});
                }
            }
            std::sort(cand.begin(), cand.end(), pair_less);
        }
        for (size_t j = 0; j < k; ++j)
        {
            const bool valid = j < take;
            out_dist[static_cast<size_t>(r) * out_stride + j] =
                valid ? cand[j].distance : std::numeric_limits<float>::infinity();
            out_label[static_cast<size_t>(r) * out_stride + j] =
                valid ? cand[j].index : std::numeric_limits<int32_t>::max();
        }
    }
}

void oracle_topk_serial(const float* in, size_t in_stride, size_t rows, size_t cols, size_t k,
                        float* out_dist, int32_t* out_label)
{
    std::vector<pair_t> row(cols);
    for (size_t r = 0; r < rows; ++r)
    {
        for (size_t c = 0; c < cols; ++c)
        {
            row[c] = pair_t{in[r * in_stride + c], static_cast<int32_t>(c)};
        }
        std::sort(row.begin(), row.end(),
                  [](const pair_t& a, const pair_t& b) { return a.distance < b.distance; });
        for (size_t j = 0; j < k; ++j)
        {
            out_dist[r * k + j] = row[j].distance;
            out_label[r * k + j] = row[j].index;
        }
    }
}

int oracle_topk_parallel(const float* in, size_t in_stride, size_t rows, size_t cols, size_t k,
                         float* out_dist, int32_t* out_label, int threads)
{
    int used = 1;
#ifdef _OPENMP
    if (threads > 0)
    {
        omp_set_num_threads(threads);
    }
    used = omp_get_max_threads();
#else
    (void)threads;
#endif
    const auto cmp = [](const pair_t& a, const pair_t& b) { return a.distance < b.distance; };
#pragma omp parallel for
    for (long long r = 0; r < static_cast<long long>(rows); ++r)
    {
        const float* row = in + static_cast<size_t>(r) * in_stride;
        std::vector<pair_t> heap(k);
        for (size_t j = 0; j < k; ++j)
        {
            heap[j] = pair_t{row[j], static_cast<int32_t>(j)};
        }
        std::make_heap(heap.begin(), heap.end(), cmp);
        for (size_t j = k; j < cols; ++j)
        {
            if (heap.front().distance > row[j])
            {
                std::pop_heap(heap.begin(), heap.end(), cmp);
                heap.back() = pair_t{row[j], static_cast<int32_t>(j)};
                std::push_heap(heap.begin(), heap.end(), cmp);
            }
        }
        std::sort(heap.begin(), heap.end(), cmp);
        for (size_t j = 0; j < k; ++j)
        {
            out_dist[static_cast<size_t>(r) * k + j] = heap[j].distance;
            out_label[static_cast<size_t>(r) * k + j] = heap[j].index;
        }
    }
    return used;
}

uint32_t oracle_checksum(const int32_t* labels, size_t k)
{
    uint32_t sink = 0;
    for (size_t j = 0; j < k; ++j)
    {
        sink += static_cast<uint32_t>(labels[j]);
    }
    return sink;
}

int oracle_verify(const float* exp_dist, const int32_t* exp_label, const float* act_dist,
                  const int32_t* act_label, size_t total, size_t k, size_t* mismatches)
{
    const float eps = 1e-3F;
    std::vector<pair_t> expected(total);
    std::vector<pair_t> actual(total);
    for (size_t i = 0; i < total; ++i)
    {
        expected[i] = pair_t{exp_dist[i], exp_label[i]};
        actual[i] = pair_t{act_dist[i], act_label[i]};
    }
    normalize(expected);
    normalize(actual);
    size_t bad = 0;
    for (size_t i = 0; i < total; ++i)
    {
        if (actual[i].index != expected[i].index)
        {
            const size_t last = i + (k - (i % k));
            if (same_distance(expected.data() + i, expected.data() + last) &&
                same_distance(actual.data() + i, actual.data() + last) &&
                approx_equal(expected[i].distance, actual[i].distance, eps))
            {
                continue;
            }
            ++bad;
        }
    }
    if (mismatches != nullptr)
    {
        *mismatches = bad;
    }
    return bad == 0 ? 1 : 0;
}

} // extern "C"
