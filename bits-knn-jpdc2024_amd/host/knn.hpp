// Algorithm plug-in interface of the `knn` driver: the phases every algorithm implements and the
// distance implementations they share.  Same phases, names and argument meaning as the
// reference's `knn` / `cuda_knn` / `cuda_distance` classes (include/bits/knn.hpp:19-129,
// cuda_knn.hpp:15-56, distance/cuda_distance.hpp:12-70, knn_args.hpp:9-37); the device work goes
// through the C ABI in bitsknn.h.
#ifndef KNN_HOST_KNN_HPP_
#define KNN_HOST_KNN_HPP_

#include <array>
#include <cstddef>
#include <cstdint>
#include <memory>
#include <string>
#include <vector>

#include "device.hpp"

enum class matrix_layout
{
    row_major,
    column_major
};

struct knn_args
{
    const float* points = nullptr;       // point matrix on the host, in points_layout
    const float* queries = nullptr;      // query matrix on the host, in queries_layout
    std::size_t point_count = 0;
    std::size_t query_count = 0;
    std::size_t dim = 0;
    matrix_layout points_layout = matrix_layout::row_major;
    matrix_layout queries_layout = matrix_layout::row_major;
    matrix_layout dist_layout = matrix_layout::row_major;
    std::size_t dist_block_size = 256;
    std::size_t selection_block_size = 256;
    std::size_t k = 1;
    std::array<std::size_t, 3> items_per_thread{1, 1, 1};
    std::size_t deg = 1;
};

struct distance_pair
{
    float distance;
    std::int32_t index;
};

// Distance matrix on the device.  prepare() uploads the vectors dim-major and allocates the
// query_count x point_count matrix, compute() fills it.
class device_distance
{
public:
    explicit device_distance(int op, std::string name) : op_(op), name_(std::move(name)) {}
    virtual ~device_distance() = default;

    virtual void prepare(const knn_args& args);
    virtual void compute();
    float transfer_seconds() const { return transfer_.seconds(); }
    float* matrix_gpu() const { return dist_.data(); }
    // copies the matrix to the host (row-major query_count x point_count)
    const std::vector<float>& matrix_cpu();
    const std::string& name() const { return name_; }

protected:
    int op_;
    std::string name_;
    knn_args args_{};
    knn_host::device_buffer<float> points_;  // in the caller's layout
    knn_host::device_buffer<float> queries_; // in the caller's layout
    knn_host::device_buffer<float> dist_;    // query_count x point_count
    knn_host::device_buffer<unsigned char> workspace_; // dim-major copies of row-major inputs
    std::vector<float> dist_host_;
    knn_host::transfer_timer transfer_;
};

std::unique_ptr<device_distance> make_l2_distance();         // `magma-dist`
std::unique_ptr<device_distance> make_partial_l2_distance(); // `magma-part-dist`
// the same values with bf16x3 products (no counterpart in the reference)
std::unique_ptr<device_distance> make_partial_l2_bf16x3_distance();
std::unique_ptr<device_distance> make_expanded_distance();   // `cublas-dist`

class knn
{
public:
    knn() = default;
    knn(const knn&) = delete;
    knn& operator=(const knn&) = delete;
    virtual ~knn() = default;

    virtual std::string id() const = 0;
    virtual void initialize(const knn_args& args);
    virtual void prepare() {}
    virtual void distances();
    virtual void selection() {}
    virtual void postprocessing() {}
    virtual std::vector<distance_pair> finish() { return {}; }
    virtual float transfer_in_seconds() const { return 0; }
    virtual float transfer_out_seconds() const { return 0; }
    void set_dist_impl(std::unique_ptr<device_distance>&& impl) { dist_impl_ = std::move(impl); }
    void no_output() { no_output_ = true; }

    std::size_t dim() const { return args_.dim; }
    std::size_t k() const { return args_.k; }
    std::size_t point_count() const { return args_.point_count; }
    std::size_t query_count() const { return args_.query_count; }

protected:
    bool no_output_ = false;
    knn_args args_{};
    std::unique_ptr<device_distance> dist_impl_;
};

// Base of the algorithms whose result lives in device memory: owns the query_count x k outputs
// and copies them back in finish().
class device_knn : public knn
{
public:
    void initialize(const knn_args& args) override;
    std::vector<distance_pair> finish() override;
    float transfer_in_seconds() const override { return dist_impl_ ? dist_impl_->transfer_seconds() : 0; }
    float transfer_out_seconds() const override { return transfer_out_.seconds(); }

protected:
    void allocate_outputs();
    float* in_dist_gpu() const { return dist_impl_->matrix_gpu(); }

    knn_host::device_buffer<float> out_dist_;
    knn_host::device_buffer<std::int32_t> out_label_;
    knn_host::transfer_timer transfer_out_;
};

// All algorithms this build registers, in the reference's order (src/main.cpp:111-155).
std::vector<std::unique_ptr<knn>> make_algorithms();

// Tie-tolerant comparison of two results (k entries per query); prints differences to stderr.
bool verify(const std::vector<distance_pair>& expected, const std::vector<distance_pair>& actual,
            std::size_t k);

#endif // KNN_HOST_KNN_HPP_
