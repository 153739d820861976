/*
 * CPU oracle for the k-NN hot path -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Plain host restatements of what the reference computes on this path, used only as the
 * checker by the parity tests, by the smoke test, and as the timed CPU baseline of the
 * benchmark.  Nothing the library ships links, loads or calls anything declared here.
 *
 * Every function names the reference source it follows (paths relative to the reference
 * tree).  How each one is pinned (golden checksums held by the reference, the reference's
 * own CUDA-free headers compiled as-is, brute force, closed forms) is listed in the header
 * comment of oracle.cpp.
 */
#ifndef BITSKNN_ORACLE_H_
#define BITSKNN_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- seeded input generation (include/bits/generator/uniform_generator.hpp:42-59,
 *      normal_generator.hpp:42-59; call order src/main.cpp:291-298) ------------------- */

/* State of the reference engine after set_seed(): minstd_rand0 seeded with `seed`, then
 * discard(4096).  seed must be non-zero (the reference draws a random seed for 0). */
uint32_t oracle_engine_init(uint64_t seed);
/* Advance an engine state by `steps` draws in O(log steps). */
uint32_t oracle_engine_skip(uint32_t state, uint64_t steps);
/* Fill out[0..count) with uniform floats in [lo, hi); returns the engine state afterwards.
 * One engine draw per value.  Uses OpenMP skip-ahead when count is large. */
uint32_t oracle_uniform_fill(uint32_t state, float lo, float hi, float* out, size_t count);
/* Fill out[0..count) with normal(mean, stddev) floats the way libstdc++'s
 * std::normal_distribution<float> does (polar method, second value cached inside one call);
 * returns the engine state afterwards. */
uint32_t oracle_normal_fill(uint32_t state, float mean, float stddev, float* out, size_t count);

/* ---- preprocessors (include/bits/preprocessor/ordering_preprocessor.hpp:36-42) ---------- */
/* descending == 0: "ascending" preprocessor; else "descending".  Zeroes all query floats and
 * sorts ALL data floats (not per vector). */
void oracle_preprocess_ordering(float* data, size_t data_floats, float* query, size_t query_floats,
                                int descending);

/* ---- CLI number parsing (include/bits/utils.hpp:20-74) ---------------------------------- */
uint64_t oracle_parse_number(const char* text);
void oracle_parse_dim3(const char* text, uint64_t out[3]);

/* ---- distances; inputs are row-major vectors (points n x d, queries q x d), output is the
 *      row-major q x n matrix ------------------------------------------------------------- */
/* squared L2 as the default distance kernel computes it: acc = fmaf(q-p, q-p, acc) over the
 * dimensions in order, fp32 (include/bits/distance/abstract_gemm.cuh:79-93). */
void oracle_dist_l2(const float* queries, const float* points, size_t q, size_t n, size_t d,
                    float* out, size_t out_stride);
/* ||p||^2 - 2 q.p (no ||q||^2): norm = fmaf(p,p,norm), dot = fmaf(q,p,dot) in dimension order,
 * result fl(norm - 2*dot) (abstract_gemm.cuh:139-169;
 * include/bits/topk/singlepass/fused_cache_kernel_structs.cuh:502-519, 622-630). */
void oracle_dist_partial_l2(const float* queries, const float* points, size_t q, size_t n, size_t d,
                            float* out, size_t out_stride);
/* fp64 ground truth of sum (q-p)^2 and of ||p||^2 - 2 q.p (selected by `partial`). */
void oracle_dist_f64(const float* queries, const float* points, size_t q, size_t n, size_t d,
                     int partial, double* out, size_t out_stride);

/* ---- top-k selection over a row-major rows x cols fp32 matrix -------------------------- */
/* Canonical result: the k smallest of each row in ascending (value, label) order, where label
 * is the column index, or labels[row*label_stride+col] when labels != NULL, plus
 * label_offsets[row] when label_offsets != NULL (bits_kernel.cuh:221-259, 317-408).
 * Values compare as IEEE floats (-0 == +0).  When k > cols the tail is (+inf, INT32_MAX). */
void oracle_topk(const float* in, size_t in_stride, const int32_t* labels, size_t label_stride,
                 const int32_t* label_offsets, size_t rows, size_t cols, size_t k,
                 float* out_dist, int32_t* out_label, size_t out_stride);
/* serial_knn restated: std::sort of every full row of (distance, index) pairs by distance
 * only, first k copied out (src/topk/serial_knn.cpp:17-54).  Order among equal distances is
 * whatever std::sort leaves. */
void oracle_topk_serial(const float* in, size_t in_stride, size_t rows, size_t cols, size_t k,
                        float* out_dist, int32_t* out_label);
/* parallel_knn::selection restated: OpenMP over rows, size-k max-heap with strict `>`
 * admission, final std::sort by distance (src/topk/parallel_knn.cpp:30-65).  `threads` <= 0
 * keeps the OpenMP default.  Returns the number of threads used. */
int oracle_topk_parallel(const float* in, size_t in_stride, size_t rows, size_t cols, size_t k,
                         float* out_dist, int32_t* out_label, int threads);

/* ---- result bookkeeping ----------------------------------------------------------------- */
/* Sum of the first k labels modulo 2^32 (src/main.cpp:410-417). */
uint32_t oracle_checksum(const int32_t* labels, size_t k);
/* verify() restated (src/verify.cpp:17-112): 1 when `actual` matches `expected` up to the
 * reordering of near-equal distances it tolerates, else 0; `mismatches` (nullable) receives
 * the count of reported differences. */
int oracle_verify(const float* exp_dist, const int32_t* exp_label, const float* act_dist,
                  const int32_t* act_label, size_t total, size_t k, size_t* mismatches);

#ifdef __cplusplus
}
#endif
#endif /* BITSKNN_ORACLE_H_ */
