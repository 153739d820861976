/*
 * Thin C-ABI shim around the reference's own CUDA-free host headers -- TEST INFRASTRUCTURE.
 *
 * It is compiled against the headers where they lie in the reference tree
 * (-I<reference>/include); no reference source is copied.  The result, oracle/_ref/libref_host.so,
 * is the real reference generator / preprocessor / number parser, used only to validate the
 * restatements in oracle.cpp.  The reference's CPU top-k and verifier cannot be built this way:
 * they include bits/knn.hpp, which pulls in <cuda_runtime.h> (and Eigen for parallel_knn).
 */
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <functional>
#include <string>
#include <vector>

#include "bits/generator/normal_generator.hpp"
#include "bits/generator/uniform_generator.hpp"
#include "bits/preprocessor/ordering_preprocessor.hpp"
#include "bits/utils.hpp"

extern "C" {

/* uniform_generator{seed, lo, hi}: generate(n, d) for the points, then generate(q, d) for the
 * queries from the same engine, as main() does. */
void ref_uniform_generate(uint64_t seed, float lo, float hi, size_t n, size_t q, size_t d,
                          float* points, float* queries)
{
    uniform_generator gen{seed, lo, hi};
    const auto p = gen.generate(n, d);
    const auto s = gen.generate(q, d);
    std::memcpy(points, p.data(), p.size() * sizeof(float));
    std::memcpy(queries, s.data(), s.size() * sizeof(float));
}

void ref_normal_generate(uint64_t seed, float mean, float stddev, size_t n, size_t q, size_t d,
                         float* points, float* queries)
{
    normal_generator gen{seed, mean, stddev};
    const auto p = gen.generate(n, d);
    const auto s = gen.generate(q, d);
    std::memcpy(points, p.data(), p.size() * sizeof(float));
    std::memcpy(queries, s.data(), s.size() * sizeof(float));
}

void ref_preprocess_ordering(float* data, size_t data_floats, float* query, size_t query_floats,
                             size_t dim, int descending)
{
    std::vector<float> d(data, data + data_floats);
    std::vector<float> s(query, query + query_floats);
    if (descending != 0)
    {
        ordering_preprocessor<std::greater<>>{}.preprocess(d, s, dim);
    }
    else
    {
        ordering_preprocessor<std::less<>>{}.preprocess(d, s, dim);
    }
    std::memcpy(data, d.data(), data_floats * sizeof(float));
    std::memcpy(query, s.data(), query_floats * sizeof(float));
}

uint64_t ref_parse_number(const char* text) { return parse_number(std::string{text}); }

void ref_parse_dim3(const char* text, uint64_t out[3])
{
    const auto r = parse_dim3(std::string{text});
    out[0] = r[0];
    out[1] = r[1];
    out[2] = r[2];
}

} // extern "C"
