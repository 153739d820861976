// What the host side of bits-fused and its kernels share: workgroup shape, kernel arguments and
// the launchers instantiated per list length.
#ifndef BITSKNN_CSRC_FUSED_ARGS_HPP_
#define BITSKNN_CSRC_FUSED_ARGS_HPP_

#include "common.hpp"

namespace bitsknn
{

constexpr int FQ_WAVES = 4;                   // waves per workgroup
constexpr int FQ_THREADS = FQ_WAVES * WAVE;   // 256
constexpr int FQ_QW = 32;                     // queries per wave (one MFMA column tile)
constexpr int FQ_QB = FQ_QW * FQ_WAVES;       // queries per workgroup
constexpr int FQ_CAP = 32;                    // buffer slots per query (= points per MFMA tile); twice
                                              // that for long lists in few dimensions, 24 of them in
                                              // LDS where three stages have to fit (fused_geometry)

// How the kernel computes: the arithmetic of the reported distances and how candidates are found.
//  FUSED_ARITH_MFMA_F32  distances from fp32 matrix instructions, every pair of a tile
//  FUSED_ARITH_BF16X3    distances from six bf16 matrix products of three pieces per operand
//  FUSED_ARITH_EXACT     a lower bound of every distance from three bf16 matrix products of two
//                        pieces per operand filters the tile; what passes is computed with
//                        sequential fused multiply-adds in dimension order (the reference's
//                        arithmetic), filtered again and appended (dimensions up to 128)
constexpr int FUSED_ARITH_MFMA_F32 = 0;
constexpr int FUSED_ARITH_BF16X3 = 1;
constexpr int FUSED_ARITH_EXACT = 2;
// (kernel-internal, 129 .. 256 dimensions of FUSED_ARITH_EXACT: the fp32 matrix instructions, on norms
// lowered by the error budget, are the filter; what passes is computed and appended as above)
constexpr int FUSED_ARITH_EXACT_F32 = 3;

constexpr int FUSED_PLAIN = -1;
constexpr int FUSED_REPEAT_MARKED = -2;
constexpr int FUSED_FIRST_RADIUS_FROM = 0;

struct fused_args
{
    const float* queries; // dim-major, stride q
    const float* points;  // dim-major, stride n
    int dim;
    int q;
    int n;
    float* out_dist;      // lists: entry i of query g in split s at ((g * splits + s) * K + i)
    std::int32_t* out_label;
    int splits;           // the points are cut into `splits` ranges, one per blockIdx.y
    int split_points;     // points per range (a multiple of 256)
    int list_stride;      // floats between the lists of consecutive (query, split) pairs: K, or more
    // A launch over a sample of the points (sample_scale > 1): every sample_scale-th stage of the
    // point matrix is visited, `visit` points in all, which are numbered 0 .. visit-1 in the
    // lists.  Otherwise visit = n, sample_scale = 1 and sample_offset = 0.
    int visit;            // points visited (the launcher sets it for a sample)
    int sample_scale;     // visited point v of a stage that starts at v0 is point
    int sample_offset;    //   v0 * sample_scale + sample_offset + (v - v0) of the matrix
    // FUSED_PLAIN: radii start from +inf.  FUSED_FIRST_RADIUS_FROM + r: the radius of query g starts
    // from final_dist[g * final_stride + r], put there by a launch over a sample; with one range of
    // points, a query whose k-th distance does not get below that value gets a NaN as its k-th
    // distance (with several ranges a range's list need not fill up, and a query that is short of k
    // distances below its first radius shows as +inf at the end of its reduced list).
    // FUSED_REPEAT_MARKED: only workgroups with a query whose k-th final distance is NaN or +inf run,
    // from +inf.
    int first_radius;
    const float* final_dist; // the caller's output array (out_dist itself with one range of points)
    int final_stride;
    // Ring of stages: a wait that is still short of its count after poll_limit polls gives up; the
    // wave then goes on (every wave leaves the kernel whatever happens), adds one to *fault at the
    // end and overwrites the k-th distances of its queries with NaN.
    int* fault;
    int poll_limit;
    // FUSED_ARITH_EXACT: the stages of the whole point matrix as they stand in LDS, one after the
    // other, written by launch_fused_image (null: the kernel cuts the points itself); image_bytes
    // below 2^31
    const void* image;
    int image_bytes;
    // queries per workgroup where the kernel has two shapes (FUSED_ARITH_EXACT up to 64 dimensions):
    // 1 = 256, else 128 (65 .. 128 dimensions: always 256)
    int workgroup;
#ifdef BITSKNN_FUSED_TIMING
    // instrumented build: cycles of all waves per phase of the stage loop, added up here
    unsigned long long* timing;
#endif
};

// one per compiled list length K (fused_inst.hip); arith: one of FUSED_ARITH_*, used where the
// dimension allows it (fp32 matrix instructions otherwise)
// the stage image of FUSED_ARITH_EXACT (stage_image.hip): its size for a point matrix of up to 64
// dimensions (0 otherwise), and the launch that writes it
size_t fused_image_bytes(int dim, int n);
// more than 256 dimensions (any_dim.hip): a plain kernel in the reference's arithmetic, one query per
// thread; takes the ranges of points of `a` (splits, split_points, list_stride), lists of k entries
hipError_t launch_fused_any_dim(const fused_args& a, int k, hipStream_t stream);
hipError_t launch_fused_image(const float* points, int dim, int n, void* image, hipStream_t stream);
hipError_t launch_fused_k_4(const fused_args& a, int arith, hipStream_t stream);
hipError_t launch_fused_k_8(const fused_args& a, int arith, hipStream_t stream);
hipError_t launch_fused_k_16(const fused_args& a, int arith, hipStream_t stream);
hipError_t launch_fused_k_32(const fused_args& a, int arith, hipStream_t stream);
hipError_t launch_fused_k_64(const fused_args& a, int arith, hipStream_t stream);
hipError_t launch_fused_k_128(const fused_args& a, int arith, hipStream_t stream);
hipError_t launch_fused_k_256(const fused_args& a, int arith, hipStream_t stream);

} // namespace bitsknn

#endif // BITSKNN_CSRC_FUSED_ARGS_HPP_
