// Comparison of two k-NN results that tolerates the freedom equal distances leave: neighbours at
// (approximately) the same distance may appear in any order, and when such a group reaches the
// end of a query's list, either result may hold different members of it.  Behaviour of the
// reference's verify() (src/verify.cpp:17-112).
#include "knn.hpp"

#include <cmath>
#include <iostream>
#include <limits>

namespace
{

constexpr float TOLERANCE = 1e-3F;

// relative comparison that degrades gracefully around zero
bool close(float a, float b)
{
    if (a == b)
    {
        return true;
    }
    const float tiny = std::numeric_limits<float>::min();
    const float magnitude = std::abs(a) + std::abs(b);
    const float gap = std::abs(a - b);
    if (a == 0 || b == 0 || magnitude < tiny)
    {
        return gap < TOLERANCE * tiny;
    }
    return gap / std::min(magnitude, std::numeric_limits<float>::max()) < TOLERANCE;
}

// inside every run of close distances, order the entries by descending index
void canonical_order(std::vector<distance_pair>& result)
{
    for (std::size_t i = 1; i < result.size(); ++i)
    {
        for (std::size_t j = i; j > 0 && close(result[j].distance, result[j - 1].distance) &&
                                result[j].index > result[j - 1].index;
             --j)
        {
            std::swap(result[j], result[j - 1]);
        }
    }
}

bool all_close(const std::vector<distance_pair>& result, std::size_t first, std::size_t last)
{
    if (first == last)
    {
        return false;
    }
    for (std::size_t i = first + 1; i < last; ++i)
    {
        if (!close(result[i - 1].distance, result[i].distance))
        {
            return false;
        }
    }
    return true;
}

} // namespace

bool verify(const std::vector<distance_pair>& expected_result,
            const std::vector<distance_pair>& actual_result, std::size_t k)
{
    std::vector<distance_pair> expected = expected_result;
    std::vector<distance_pair> actual = actual_result;
    canonical_order(expected);
    canonical_order(actual);
    bool same = true;
    for (std::size_t i = 0; i < expected.size() && i < actual.size(); ++i)
    {
        if (actual[i].index == expected[i].index)
        {
            continue;
        }
        const std::size_t row_end = i - (i % k) + k;
        const bool boundary_tie = all_close(expected, i, row_end) && all_close(actual, i, row_end) &&
                                  close(expected[i].distance, actual[i].distance);
        if (boundary_tie)
        {
            continue;
        }
        std::cerr << "Difference at index " << i << " (expected: " << expected[i].index
                  << ", actual: " << actual[i].index << ")" << '\n';
        std::cerr << "- expected distance: " << expected[i].distance << '\n';
        std::cerr << "- actual distance: " << actual[i].distance << '\n';
        same = false;
    }
    return same;
}
