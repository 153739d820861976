// Test-only driver of the `knn` binary's verify() (host/verify.cpp): reads two results from
// stdin and prints 1 when verify() accepts them, else 0 (its reports go to stderr).
// Input: k, total, then `total` (distance, index) pairs of the expected result and `total` of the
// actual one.
#include "knn.hpp"

#include <cstdio>
#include <iostream>
#include <vector>

int main()
{
    std::size_t k = 0;
    std::size_t total = 0;
    if (!(std::cin >> k >> total))
    {
        return 2;
    }
    std::vector<distance_pair> expected(total);
    std::vector<distance_pair> actual(total);
    for (auto* result : {&expected, &actual})
    {
        for (auto& pair : *result)
        {
            if (!(std::cin >> pair.distance >> pair.index))
            {
                return 2;
            }
        }
    }
    std::printf("%d\n", verify(expected, actual, k) ? 1 : 0);
    return 0;
}
