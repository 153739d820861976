/*
 * bitsknn -- C ABI of the MI355X (gfx950) k-NN hot path.
 *
 * Plain C, raw device pointers and sizes.  Every entry point
 *   - returns 0 (BITSKNN_OK) or a BITSKNN_ERR_* code; the message of the last failure on the
 *     calling thread is available from bitsknn_last_error();
 *   - takes device pointers that the caller owns, allocates nothing and frees nothing;
 *   - enqueues its kernels on `stream` (a hipStream_t passed as void*, NULL = default stream)
 *     and returns without synchronising -- the caller synchronises, like the reference's host
 *     wrappers do at the end of every phase (reference src/topk/singlepass/bits_knn.cu:95,
 *     src/knn.cpp:28).
 *
 * Each declaration cites the reference interface it replaces (paths relative to the
 * reference tree).  Strides are in elements, not bytes.
 */
#ifndef BITSKNN_H_
#define BITSKNN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BITSKNN_OK 0
#define BITSKNN_ERR_UNSUPPORTED 1 /* parameter outside the compiled lists (reference: runtime_error "Unsupported ...") */
#define BITSKNN_ERR_INVALID 2     /* null pointer / inconsistent sizes */
#define BITSKNN_ERR_HIP 3         /* a HIP runtime call failed (reference: CUCH -> runtime_error) */
#define BITSKNN_ERR_INTERNAL 4    /* a kernel reported that it could not keep its own protocol (bitsknn_fused_status) */

/* Message of the last error reported on this thread ("" if none). Never NULL. */
const char* bitsknn_last_error(void);

/* Library version string. */
const char* bitsknn_version(void);

/*
 * bits top-k selection: for every row of a rows x cols fp32 matrix, the k smallest values in
 * ascending order with their labels; equal values are ordered by lower label.
 *
 * Replaces run_bits_kernel<float, int32_t, PREFETCH, BLOCK_SIZE, BATCH_SIZE, K>
 * (include/bits/topk/singlepass/bits_kernel.hpp:22-27,
 *  include/bits/topk/singlepass/detail/bits_kernel.cuh:317-429) and the runtime dispatch of
 * struct bits (src/topk/singlepass/bits_knn.cu:29-65).
 *
 *  in, in_row_stride       distance matrix, row r starts at in + r*in_row_stride
 *  in_label                NULL: the label of column c is c; else a rows x cols int32 matrix
 *  label_row_stride        row stride of in_label (ignored when in_label is NULL)
 *  label_offsets           NULL or rows int32 values added to every label of that row
 *  out_dist, out_label     rows x k outputs, row stride out_row_stride (>= k)
 *  k                       1 <= k <= 2048; rounded up to the next of {16,...,2048} internally
 *  block_size              threads per row: 128, 256 or 512
 *  items_per_thread        values each thread has in flight per iteration: 1..16
 *  prefetch                non-zero (the reference's `bits-prefetch`): twice as many values in
 *                          flight per thread, i.e. the next batch is requested together with the
 *                          current one; zero: `bits`
 *
 * Errors: "Unsupported block size: N", "Unsupported batch size: N", "Unsupported k value: N"
 * exactly as the reference throws them (bits_knn.cu:52-62).
 * When k > cols the tail of a row is filled with (+inf, INT32_MAX).
 */
int bitsknn_topk_bits_f32(const float* in, size_t in_row_stride, const int32_t* in_label,
                          size_t label_row_stride, const int32_t* label_offsets, size_t rows,
                          size_t cols, float* out_dist, int32_t* out_label, size_t out_row_stride,
                          uint32_t k, uint32_t block_size, uint32_t items_per_thread, int prefetch,
                          void* stream);

/*
 * bits-sq: bits top-k for few, long rows.  Every row of the contiguous rows x cols matrix is cut
 * into `parts` equal parts that are selected by separate workgroups (labels shifted by the part's
 * first column), and the parts * k pairs of a row are selected again with their labels.  Same
 * result as bitsknn_topk_bits_f32 on the whole rows, bit for bit.
 *
 * Replaces single_query_bits::selection (src/topk/singlepass/bits_knn.cu:132-186: two launches of
 * the bits kernel, the prefetching form, and populate_label_offsets_kernel :67-76).  The labels of
 * a part are shifted inside the kernel.  With up to 1024 parts in all it is one launch: the
 * workgroup that finishes the last part of a row (a counter per row in device memory) selects from
 * the row's pairs itself.  With more parts, or where the pairs of a row would not start on a
 * 16-byte boundary (parts * k not a multiple of 4), the second pass is a launch of its own.
 *
 *  in                     rows x cols, row stride cols; cols a multiple of parts
 *  parts                  parts per row (1: as bitsknn_topk_bits_f32 with prefetch)
 *  part_dist, part_label  rows * parts * k pairs of device memory for the parts' results
 *  counters               rows int32 in device memory, zero before the first call; every call
 *                         leaves them zero
 *  out_dist, out_label    rows x k outputs, row stride out_row_stride (>= k)
 *  k, block_size, items_per_thread as for bitsknn_topk_bits_f32, with its messages.
 */
int bitsknn_topk_bits_parts_f32(const float* in, size_t rows, size_t cols, uint32_t parts,
                                float* part_dist, int32_t* part_label, int32_t* counters,
                                float* out_dist, int32_t* out_label, size_t out_row_stride, uint32_t k,
                                uint32_t block_size, uint32_t items_per_thread, void* stream);

/*
 * partial-bitonic-regs: top-k of every row by sorting the row block after block in registers and
 * merging each sorted block into the running result, with no filtering of the input (the
 * baseline that the bits kernel's buffer and filter are measured against).  Same matrix and
 * output layout and the same ordering of equal values as bitsknn_topk_bits_f32; labels are
 * column indices.
 *
 * Replaces partial_bitonic_regs_kernel<K, BLOCK_SIZE> and partial_bitonic_regs_run
 * (src/topk/singlepass/partial_bitonic.cu:217-294, 341-358).
 *  block_size  one of 64, 128, 256, 512 ("Unsupported block size: N" otherwise)
 *  k           1..2048                   ("Unsupported k value: N" otherwise)
 */
int bitsknn_topk_partial_bitonic_f32(const float* in, size_t in_row_stride, size_t rows, size_t cols,
                                     float* out_dist, int32_t* out_label, size_t out_row_stride,
                                     uint32_t k, uint32_t block_size, void* stream);

/*
 * Label offsets for a row-split single-query problem: offsets[i] = (i % parts) * cols_per_part
 * for i < rows*parts.  Replaces populate_label_offsets_kernel
 * (src/topk/singlepass/bits_knn.cu:67-76).
 */
int bitsknn_label_offsets(int32_t* offsets, size_t rows, size_t parts, size_t cols_per_part,
                          void* stream);

/* Fill count floats with value.  Replaces fill_kernel (src/cuda_stream.cu:9-24). */
int bitsknn_fill_f32(float* dst, size_t count, float value, void* stream);

/*
 * Calibration: the minimum of every row of a rows x cols fp32 matrix by a plain streaming read with
 * the row-per-workgroup mapping and the 16-byte non-temporal loads of the top-k kernel and no
 * other work.  Its rate is the read rate such a kernel can reach on the machine at hand, the
 * yardstick next to the published HBM peak.  No counterpart in the reference.
 * Rows must start on 16-byte boundaries (BITSKNN_ERR_INVALID otherwise).
 */
int bitsknn_stream_read_f32(const float* in, size_t in_row_stride, size_t rows, size_t cols,
                            float* row_min, void* stream);

/*
 * Distance matrix dist[i*dist_row_stride + j] between query i and point j, inputs dim-major
 * (component t of vector v at base[t*stride + v]), as the reference uploads them
 * (src/distance/magma_distance.cu:13-71).
 *
 * Replaces run_abstract_gemm<Ops>(K, M, N, A, B, C)
 * (include/bits/distance/abstract_gemm.cuh:730-755) for
 *   BITSKNN_DIST_L2          Ops = l2_ops: acc = fmaf(q-p, q-p, acc) over the dimensions in
 *                            order (abstract_gemm.cuh:59-100); bit-reproducible
 *   BITSKNN_DIST_PARTIAL_L2  Ops = partial_l2_ops: ||p||^2 - 2 q.p, no ||q||^2
 *                            (abstract_gemm.cuh:108-170); contraction on fp32 MFMA
 * and the SGEMM + squared_length_kernel + add_norm_kernel sequence of
 * cublas_distance::compute (src/distance/cublas_distance.cu:111-186) for
 *   BITSKNN_DIST_EXPANDED    -2 q.p on fp32 MFMA, then + ||p||^2, written once
 * No counterpart in the reference:
 *   BITSKNN_DIST_PARTIAL_L2_BF16X3  the values of BITSKNN_DIST_PARTIAL_L2 with every fp32 operand
 *                            cut exactly into three bf16 pieces and a product taken as the fp32
 *                            sum of six bf16 matrix products (what is left out is below 2^-23 of
 *                            a product); for dimensions 33 .. 64 and matrix rows that start on
 *                            16-byte boundaries, otherwise the same as BITSKNN_DIST_PARTIAL_L2
 */
#define BITSKNN_DIST_L2 0
#define BITSKNN_DIST_PARTIAL_L2 1
#define BITSKNN_DIST_EXPANDED 2
#define BITSKNN_DIST_PARTIAL_L2_BF16X3 3
int bitsknn_dist_f32(int op, int dim, size_t q, size_t n, const float* queries_dim_major,
                     size_t query_stride, const float* points_dim_major, size_t point_stride,
                     float* dist, size_t dist_row_stride, void* stream);

/*
 * bitsknn_dist_f32 for vectors in the caller's layout.  The reference's distance classes take the
 * points and the queries in either matrix layout of knn_args, four combinations
 * (src/distance/cublas_distance.cu:122-149: the transposition flags of the SGEMM and the
 * row_major / column_major forms of squared_length_kernel :23-60; include/bits/layout.hpp:4):
 *   BITSKNN_LAYOUT_ROW_MAJOR     the vectors one after the other: component t of vector v at
 *                                base[v*stride + t], stride >= dim (matrix_layout::row_major)
 *   BITSKNN_LAYOUT_COLUMN_MAJOR  dim-major as for bitsknn_dist_f32: base[t*stride + v], stride >=
 *                                the vector count (matrix_layout::column_major)
 * A set of vectors given one after the other is first brought into dim-major form on the device
 * (a copy in `workspace`, 16-byte aligned, bitsknn_dist_layout_workspace_bytes() bytes: dim x the
 * count rounded up to a multiple of four floats per such set; nothing for dim-major sets), then
 * the kernels of bitsknn_dist_f32 run: same values bit for bit in every combination.
 * Errors as for bitsknn_dist_f32, plus BITSKNN_ERR_INVALID for an unknown layout or a workspace
 * that is missing, misaligned or too small.
 */
#define BITSKNN_LAYOUT_ROW_MAJOR 0
#define BITSKNN_LAYOUT_COLUMN_MAJOR 1
size_t bitsknn_dist_layout_workspace_bytes(int dim, size_t q, size_t n, int queries_layout,
                                           int points_layout);
int bitsknn_dist_layout_f32(int op, int dim, size_t q, size_t n, const float* queries,
                            int queries_layout, size_t query_stride, const float* points,
                            int points_layout, size_t point_stride, float* dist, size_t dist_row_stride,
                            void* workspace, size_t workspace_bytes, void* stream);

/*
 * bits-fused: partial squared L2 distance (||p||^2 - 2 q.p) and top-k in one kernel; the
 * q x n distance matrix is never written to memory.  Outputs q x k, row stride k, ascending,
 * equal distances ordered by lower point index.
 *
 * Replaces fused_cache::run / launch_fused_cache
 * (src/topk/singlepass/fused_cache_knn.cu:29-145,
 *  include/bits/topk/singlepass/detail/fused_cache_kernel.cuh:25-42).
 * Inputs dim-major with strides q and n (fused_cache_knn.cu:156-194).
 *  k                          one of 4, 8, 16, 32, 64, 128, 256 ("Unsupported k value: N" otherwise)
 *  query_reg, db_reg, dim_reg, block_query_dim, dim_mult
 *                             the reference's tuning parameters; validated against its lists
 *                             ({2,4,8,16}, {4,8,16}, {1,2,4}, {1,2,4}, {1,2,4}) with its
 *                             messages; dim must be >= dim_mult*dim_reg as there.  Accepted for
 *                             compatibility only: they describe a register tiling for the fp32
 *                             vector unit and do not change the matrix-core kernel, so a sweep
 *                             over them measures the same kernel every time (what a sweep can
 *                             vary here: bitsknn_fused_l2_topk_f32_tuned)
 * The distances are computed in the reference's arithmetic (BITSKNN_FUSED_EXACT below) in every
 * dimension.  More than 256 dimensions (the reference's kernel has only a lower bound on the
 * dimension, fused_cache_knn.cu:63-67) are served by a plain kernel on the vector unit, one query
 * per thread: correct and bit-identical, not tuned.
 * A call enqueues one to three kernels on `stream` (long lists over many points are preceded by a
 * pass over a sample of the points, which gives every query a first radius, and followed by one
 * that repeats the queries whose first radius proved too low); until the last of them has run,
 * out_dist and out_label hold intermediate lists.  A NaN or infinite distance is never reported
 * as a neighbour before a finite one.
 */
int bitsknn_fused_l2_topk_f32(const float* queries_dim_major, const float* points_dim_major,
                              int dim, int32_t q, int32_t n, float* out_dist, int32_t* out_label,
                              int k, int query_reg, int db_reg, int dim_reg, int block_query_dim,
                              int dim_mult, void* stream);

/*
 * bits-fused with a caller-provided workspace.  Same neighbours as bitsknn_fused_l2_topk_f32, and
 * still the fused kernel: no distance is written to memory.  When there are too few queries to
 * fill the GPU with one workgroup per 128 queries, the points are cut into ranges that are
 * searched by separate workgroups; their partial lists (k pairs per query and range) go to the
 * workspace and a bits pass (explicit labels) selects the final k.  Same lists bit for bit.
 *
 * No counterpart in the reference, whose fused kernel always runs one thread block per query tile
 * (src/topk/singlepass/fused_cache_knn.cu:60-69); the host wrapper that owns the device memory
 * (fused_cache_knn::initialize, fused_cache_knn.cu:149-195) is where the workspace is allocated.
 *
 * bitsknn_fused_workspace_bytes returns the size the call wants: 8*q*ranges*k bytes, at most 64
 * ranges; 0 when the queries fill the GPU by themselves.  A smaller workspace (4-byte aligned) is
 * not an error: the call uses as many ranges as fit, down to the single kernel without any.
 *
 * The stage image.  In the exact arithmetic every workgroup cuts every point into bf16
 * pieces again.  With bitsknn_fused_image_bytes(dim, n) more bytes in the workspace, behind the
 * partial lists rounded up to a multiple of 256 bytes (and the workspace 16-byte aligned), a launch
 * of its own writes the stages of the whole point matrix there once per call and the fused kernel
 * copies them (65536 queries x 2^20 points, k = 32: d = 8 7.4 -> 7.1 ms, d = 16 9.9 -> 9.6 ms).  It is
 * written from 4096 queries on in up to 16 dimensions (bitsknn_fused_tuning::image overrides that);
 * the results are the same bit for bit with and without it.  bitsknn_fused_image_bytes is 0 where no image is used
 * (dim > 64, or an image of 2 GiB and more).
 * Errors as for bitsknn_fused_l2_topk_f32.
 */
size_t bitsknn_fused_workspace_bytes(int32_t q, int32_t n, int k);
size_t bitsknn_fused_image_bytes(int dim, int32_t n);
int bitsknn_fused_l2_topk_f32_ws(const float* queries_dim_major, const float* points_dim_major,
                                 int dim, int32_t q, int32_t n, float* out_dist, int32_t* out_label,
                                 int k, int query_reg, int db_reg, int dim_reg, int block_query_dim,
                                 int dim_mult, void* workspace, size_t workspace_bytes, void* stream);

/*
 * bits-fused with the arithmetic of the products q.p chosen per call (nothing process-wide is
 * read); workspace may be NULL (then as bitsknn_fused_l2_topk_f32) or as for
 * bitsknn_fused_l2_topk_f32_ws.
 *   BITSKNN_FUSED_EXACT   what the entry points above use.  Every reported distance
 *                         is computed as the reference's kernel computes it -- norm and dot
 *                         product by sequential fused multiply-adds over the dimensions in order,
 *                         then norm - 2 dot (include/bits/topk/singlepass/
 *                         fused_cache_kernel_structs.cuh:457-522, :622-631) -- so the lists equal
 *                         the reference arithmetic's bit for bit, equal distances by lower index.
 *                         Which pairs to compute is decided by a filter on the bf16 matrix
 *                         instructions (v_mfma_f32_32x32x16_bf16, two bf16 pieces per operand, three
 *                         products) whose value is a guaranteed lower bound of the distance less a
 *                         slack of 2^-13 ||q||^2 (1.5 * 2^-13 above 64 dimensions): no pair below a
 *                         query's current k-th distance is ever dropped.  In 129 to 256
 *                         dimensions the fp32 matrix instructions (on norms lowered by the same
 *                         budget) are that filter: 1 to 3 times the time of BITSKNN_FUSED_FP32
 *                         there, which callers who do not need the reference's bits can ask for.
 *   BITSKNN_FUSED_FP32    every distance from fp32 matrix instructions (v_mfma_f32_32x32x2_f32):
 *                         within 1e-5 of the reference arithmetic, not bit-identical to it.
 *   BITSKNN_FUSED_BF16X3  for 9 <= dim <= 64: every fp32 operand is cut exactly into three bf16
 *                         pieces and a product is the fp32 sum of six bf16 products on the bf16
 *                         matrix path; what is left out is below 2^-23 of a product, the size of
 *                         one fp32 rounding.  Other dimensions use BITSKNN_FUSED_FP32.
 *   (More than 256 dimensions: whatever the value, the plain kernel in the reference's arithmetic.)
 * The reference's fused kernel multiplies on the fp32 vector unit
 * (fused_cache_kernel_structs.cuh:457-522); the last two have no counterpart there.
 * BITSKNN_ERR_INVALID for another value of `arithmetic`.
 */
#define BITSKNN_FUSED_FP32 0
#define BITSKNN_FUSED_BF16X3 1
#define BITSKNN_FUSED_EXACT 2
int bitsknn_fused_l2_topk_f32_ex(const float* queries_dim_major, const float* points_dim_major,
                                 int dim, int32_t q, int32_t n, float* out_dist, int32_t* out_label,
                                 int k, int query_reg, int db_reg, int dim_reg, int block_query_dim,
                                 int dim_mult, int arithmetic, void* workspace, size_t workspace_bytes,
                                 void* stream);

/*
 * bits-fused with the launch parameters of this implementation in the caller's hands: what a tuning
 * sweep varies here.  The reference tunes its fused kernel over a register tiling (QUERY_REG,
 * DB_REG, DIM_REG, BLOCK_QUERY_DIM, DIM_MULT: src/topk/singlepass/fused_cache_knn.cu:39-145,
 * scripts/run-fused-cache-params.sh); the matrix-core kernels here have no such tiling to choose,
 * and what does change their time is chosen per call by rules measured on one machine:
 *   arithmetic    as for bitsknn_fused_l2_topk_f32_ex (the plain entry points take
 *                 BITSKNN_FUSED_EXACT)
 *   ranges        how many ranges the points are cut into (separate workgroups per range, partial
 *                 lists of 8*q*ranges*k bytes in the workspace, one bits pass at the end); 0 = the
 *                 library's choice (enough workgroups for two per compute unit -- one in 129 to
 *                 256 dimensions of BITSKNN_FUSED_EXACT, where a unit holds one --, at most 64); fewer
 *                 are used when the workspace is smaller or the ranges would fall below 256 points
 *   first_radius  whether the lists start from radii taken from a launch over a sample of the points
 *                 (one stage in every first_radius, 2 .. 4096; -1: never; 0: the library's choice,
 *                 lists of 128 and more on at least 2^17 points, of 64 and more over ranges); a
 *                 sample whose lists would not reach the rank the guarantee needs is not taken
 *   image         whether the points are cut into the stages of BITSKNN_FUSED_EXACT once, into the
 *                 workspace behind the partial lists (bitsknn_fused_image_bytes), instead of by
 *                 every workgroup again: 1 = whenever the workspace has room, -1 = never, 0 = the
 *                 library's choice (from 4096 queries on, up to 16 dimensions)
 *   workgroup     queries per workgroup where the kernel comes in two shapes (BITSKNN_FUSED_EXACT up
 *                 to 64 dimensions; 65 .. 128 dimensions have the one of 256 queries only and
 *                 ignore the field): 128 (four waves), 256 (eight waves sharing stages of twice
 *                 the points; no stage image then) or 0 = the library's choice (256 where
 *                 ceil(q / 256) * ranges workgroups, one at a time on each of the 256 compute
 *                 units, leave at most an eighth of the units idle in their last round; lists of
 *                 64 and more only over one range of points, the longer ones in more dimensions)
 * tuning == NULL: the library's choices.  Results do not depend on the tuning (for
 * BITSKNN_FUSED_EXACT bit for bit; for the other arithmetics the distances of a point can differ in
 * the last bit between one range and several).  bitsknn/tuning.py sweeps these and records the
 * best per problem.  Errors as for bitsknn_fused_l2_topk_f32_ex, plus BITSKNN_ERR_INVALID for
 * values outside the ranges above or non-zero reserved words.
 */
typedef struct bitsknn_fused_tuning
{
    int32_t ranges;
    int32_t first_radius;
    int32_t image;
    int32_t workgroup;
    int32_t reserved[4];
} bitsknn_fused_tuning;
int bitsknn_fused_l2_topk_f32_tuned(const float* queries_dim_major, const float* points_dim_major,
                                    int dim, int32_t q, int32_t n, float* out_dist, int32_t* out_label,
                                    int k, int arithmetic, const bitsknn_fused_tuning* tuning,
                                    void* workspace, size_t workspace_bytes, void* stream);

/*
 * bitsknn_fused_l2_topk_f32_ws for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc): the partial lists go to
 * scratch memory inside the library, a static device array of bitsknn_fused_static_scratch_bytes()
 * = 32 MiB that every GPU the library runs on holds until the process ends.  The call allocates
 * and frees nothing (its first call on a device looks up the array's address on that device).
 * Same results as bitsknn_fused_l2_topk_f32_ws with the workspace it asks for, bit for bit.
 *
 * No counterpart in the reference.
 *
 * Errors as for bitsknn_fused_l2_topk_f32, plus BITSKNN_ERR_INVALID when
 * bitsknn_fused_workspace_bytes(q, n, k) exceeds the scratch memory (nothing is launched then).
 * All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (different
 * streams or threads) race on it and must be serialised by the caller.
 */
size_t bitsknn_fused_static_scratch_bytes(void);
int bitsknn_fused_l2_topk_f32_static(const float* queries_dim_major, const float* points_dim_major,
                                     int dim, int32_t q, int32_t n, float* out_dist,
                                     int32_t* out_label, int k, int query_reg, int db_reg, int dim_reg,
                                     int block_query_dim, int dim_mult, void* stream);

/*
 * Health check of the bits-fused kernels on the current device.  Where the stages of points are
 * handed from wave to wave through counters in LDS instead of barriers, a wave waits for a stage
 * with a bounded number of polls, so that every wave leaves the kernel whatever happens.  The
 * bound is never reached in a correct run; if it is, the wave goes on with what it has, writes NaN
 * as the k-th distance of each of its queries and counts the event in a word of device memory
 * inside the library.  This call synchronises `stream`, reads that word and clears it: BITSKNN_OK
 * when no wait has run out of polls since the last check, else BITSKNN_ERR_INTERNAL (the results
 * of the fused calls since the last check must be discarded).  The `knn` driver checks after every
 * fused selection, where the reference synchronises and checks its launch
 * (src/topk/singlepass/fused_cache_knn.cu:213-215, CUCH(cudaGetLastError()) in
 * include/bits/topk/singlepass/detail/fused_cache_kernel.cuh:38-42).
 * BITSKNN_FUSED_POLL_LIMIT in the environment (read once per process, 0 .. 4194304, default
 * 4194304) sets the bound; tests set it to 0 to reach this path with kernels that still end
 * normally.
 */
int bitsknn_fused_status(void* stream);

#ifdef __cplusplus
}
#endif
#endif /* BITSKNN_H_ */
