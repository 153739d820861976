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
                                              // that for long lists in few dimensions (fused_geometry)

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
};

// one per compiled list length K (fused_inst.hip); split: products from three bf16 pieces per
// operand where the dimension allows it
hipError_t launch_fused_k_4(const fused_args& a, bool split, hipStream_t stream);
hipError_t launch_fused_k_8(const fused_args& a, bool split, hipStream_t stream);
hipError_t launch_fused_k_16(const fused_args& a, bool split, hipStream_t stream);
hipError_t launch_fused_k_32(const fused_args& a, bool split, hipStream_t stream);
hipError_t launch_fused_k_64(const fused_args& a, bool split, hipStream_t stream);
hipError_t launch_fused_k_128(const fused_args& a, bool split, hipStream_t stream);
hipError_t launch_fused_k_256(const fused_args& a, bool split, hipStream_t stream);

} // namespace bitsknn

#endif // BITSKNN_CSRC_FUSED_ARGS_HPP_
