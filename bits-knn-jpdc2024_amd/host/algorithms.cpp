// Algorithms registered in the `knn` driver.  Each one mirrors the phases of its reference
// counterpart (cited per class); all device work goes through the C ABI in bitsknn.h.
#include "knn.hpp"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <stdexcept>
#include <utility>

namespace
{

using knn_host::device_buffer;
using knn_host::sync_default_stream;

// dim-major copy (component t of vector v at [t*count + v]) of a matrix given in `layout`
std::vector<float> to_dim_major(const float* data, std::size_t count, std::size_t dim,
                                matrix_layout layout)
{
    std::vector<float> out(count * dim);
    if (layout == matrix_layout::column_major)
    {
        std::copy(data, data + count * dim, out.begin());
        return out;
    }
    for (std::size_t v = 0; v < count; ++v)
    {
        for (std::size_t t = 0; t < dim; ++t)
        {
            out[t * count + v] = data[v * dim + t];
        }
    }
    return out;
}

int layout_code(matrix_layout layout)
{
    return layout == matrix_layout::row_major ? BITSKNN_LAYOUT_ROW_MAJOR : BITSKNN_LAYOUT_COLUMN_MAJOR;
}

float component(const float* data, std::size_t count, std::size_t dim, matrix_layout layout,
                std::size_t v, std::size_t t)
{
    return layout == matrix_layout::row_major ? data[v * dim + t] : data[t * count + v];
}

} // namespace

// ---------------------------------------------------------------------------------------------
// distances (reference: src/distance/magma_distance.cu:13-103, cublas_distance.cu:104-186)
// ---------------------------------------------------------------------------------------------

void device_distance::prepare(const knn_args& args)
{
    args_ = args;
    if (args_.dist_layout != matrix_layout::row_major)
    {
        throw std::runtime_error{"Only the row-major layout of the distance matrix is supported."};
    }
    // the vectors go to the device in the caller's layout (reference: cuda_distance::prepare,
    // src/distance/cuda_distance.cpp; the layouts are resolved on the device)
    points_ = device_buffer<float>{args_.dim * args_.point_count};
    queries_ = device_buffer<float>{args_.dim * args_.query_count};
    dist_ = device_buffer<float>{args_.query_count * args_.point_count};
    workspace_ = device_buffer<unsigned char>{bitsknn_dist_layout_workspace_bytes(
        static_cast<int>(args_.dim), args_.query_count, args_.point_count, layout_code(args_.queries_layout),
        layout_code(args_.points_layout))};
    transfer_.start();
    points_.upload(args_.points, points_.size());
    queries_.upload(args_.queries, queries_.size());
    sync_default_stream();
    transfer_.stop();
}

void device_distance::compute()
{
    const bool q_rows = args_.queries_layout == matrix_layout::row_major;
    const bool p_rows = args_.points_layout == matrix_layout::row_major;
    BITSKNN_CHECK(bitsknn_dist_layout_f32(
        op_, static_cast<int>(args_.dim), args_.query_count, args_.point_count, queries_.data(),
        layout_code(args_.queries_layout), q_rows ? args_.dim : args_.query_count, points_.data(),
        layout_code(args_.points_layout), p_rows ? args_.dim : args_.point_count, dist_.data(), args_.point_count,
        workspace_.size() != 0 ? workspace_.data() : nullptr, workspace_.size(), nullptr));
}

const std::vector<float>& device_distance::matrix_cpu()
{
    dist_host_.resize(dist_.size());
    dist_.download(dist_host_.data(), dist_host_.size());
    sync_default_stream();
    return dist_host_;
}

std::unique_ptr<device_distance> make_l2_distance()
{
    return std::make_unique<device_distance>(BITSKNN_DIST_L2, "magma-dist");
}

std::unique_ptr<device_distance> make_partial_l2_distance()
{
    return std::make_unique<device_distance>(BITSKNN_DIST_PARTIAL_L2, "magma-part-dist");
}

std::unique_ptr<device_distance> make_partial_l2_bf16x3_distance()
{
    return std::make_unique<device_distance>(BITSKNN_DIST_PARTIAL_L2_BF16X3, "magma-part-dist-bf16x3");
}

std::unique_ptr<device_distance> make_expanded_distance()
{
    return std::make_unique<device_distance>(BITSKNN_DIST_EXPANDED, "cublas-dist");
}

// ---------------------------------------------------------------------------------------------
// base classes (reference: src/knn.cpp:11-31, src/cuda_knn.cpp:12-63)
// ---------------------------------------------------------------------------------------------

void knn::initialize(const knn_args& args)
{
    args_ = args;
    args_.dist_layout = matrix_layout::row_major;
    if (dist_impl_ == nullptr)
    {
        dist_impl_ = make_l2_distance(); // the default distance of every algorithm
    }
    dist_impl_->prepare(args_);
}

void knn::distances()
{
    dist_impl_->compute();
    sync_default_stream();
}

void device_knn::allocate_outputs()
{
    out_dist_ = device_buffer<float>{query_count() * k()};
    out_label_ = device_buffer<std::int32_t>{query_count() * k()};
}

void device_knn::initialize(const knn_args& args)
{
    knn::initialize(args);
    allocate_outputs();
}

std::vector<distance_pair> device_knn::finish()
{
    if (no_output_)
    {
        transfer_out_.start();
        transfer_out_.stop();
        return {};
    }
    const std::size_t total = query_count() * k();
    std::vector<float> dist(total);
    std::vector<std::int32_t> label(total);
    transfer_out_.start();
    out_dist_.download(dist.data(), total);
    out_label_.download(label.data(), total);
    sync_default_stream();
    transfer_out_.stop();
    std::vector<distance_pair> result(total);
    for (std::size_t i = 0; i < total; ++i)
    {
        result[i] = distance_pair{dist[i], label[i]};
    }
    return result;
}

namespace
{

// ---------------------------------------------------------------------------------------------
// CPU reference algorithms (reference: src/topk/serial_knn.cpp:10-54, parallel_knn.cpp:12-67)
// ---------------------------------------------------------------------------------------------

// Full sort of every row of the device-computed distance matrix, by distance only.
class serial_knn : public knn
{
public:
    std::string id() const override { return "serial"; }

    void prepare() override
    {
        rows_.clear();
        rows_.reserve(point_count() * query_count());
    }

    void distances() override
    {
        knn::distances();
        const auto& matrix = dist_impl_->matrix_cpu();
        rows_.clear();
        for (std::size_t i = 0; i < query_count(); ++i)
        {
            for (std::size_t j = 0; j < point_count(); ++j)
            {
                rows_.push_back(distance_pair{matrix[i * point_count() + j], static_cast<std::int32_t>(j)});
            }
        }
    }

    void selection() override
    {
        for (std::size_t i = 0; i < query_count(); ++i)
        {
            const auto first = rows_.begin() + static_cast<std::ptrdiff_t>(i * point_count());
            std::sort(first, first + static_cast<std::ptrdiff_t>(point_count()),
                      [](const distance_pair& a, const distance_pair& b) { return a.distance < b.distance; });
        }
    }

    std::vector<distance_pair> finish() override
    {
        std::vector<distance_pair> result(query_count() * k());
        for (std::size_t i = 0; i < query_count(); ++i)
        {
            std::copy_n(rows_.begin() + static_cast<std::ptrdiff_t>(i * point_count()), k(),
                        result.begin() + static_cast<std::ptrdiff_t>(i * k()));
        }
        return result;
    }

private:
    std::vector<distance_pair> rows_;
};

// OpenMP over the queries: size-k max-heap with strict admission, then a final sort.  The
// distances (||p||^2 - 2 q.p, the quantity the reference's CPU distance computes with Eigen) are
// computed on the host as well.
class parallel_knn : public knn
{
public:
    std::string id() const override { return "parallel"; }

    void initialize(const knn_args& args) override
    {
        args_ = args;
        args_.dist_layout = matrix_layout::row_major;
    }

    void prepare() override
    {
        result_.clear();
        result_.resize(query_count() * k());
    }

    void distances() override
    {
        const std::size_t n = point_count();
        const std::size_t q = query_count();
        const std::size_t d = dim();
        matrix_.resize(q * n);
        std::vector<float> norm(n, 0.0F);
        for (std::size_t j = 0; j < n; ++j)
        {
            for (std::size_t t = 0; t < d; ++t)
            {
                const float p = component(args_.points, n, d, args_.points_layout, j, t);
                norm[j] += p * p;
            }
        }
#pragma omp parallel for
        for (std::size_t i = 0; i < q; ++i)
        {
            for (std::size_t j = 0; j < n; ++j)
            {
                float dot = 0;
                for (std::size_t t = 0; t < d; ++t)
                {
                    dot += component(args_.queries, q, d, args_.queries_layout, i, t) *
                           component(args_.points, n, d, args_.points_layout, j, t);
                }
                matrix_[i * n + j] = norm[j] - 2 * dot;
            }
        }
    }

    void selection() override
    {
        const auto less = [](const distance_pair& a, const distance_pair& b) { return a.distance < b.distance; };
        const std::size_t n = point_count();
        const std::size_t kk = k();
#pragma omp parallel for
        for (std::size_t i = 0; i < query_count(); ++i)
        {
            const float* row = matrix_.data() + i * n;
            const auto heap_begin = result_.begin() + static_cast<std::ptrdiff_t>(i * kk);
            const auto heap_end = heap_begin + static_cast<std::ptrdiff_t>(kk);
            for (std::size_t j = 0; j < kk; ++j)
            {
                heap_begin[static_cast<std::ptrdiff_t>(j)] = distance_pair{row[j], static_cast<std::int32_t>(j)};
            }
            std::make_heap(heap_begin, heap_end, less);
            for (std::size_t j = kk; j < n; ++j)
            {
                if (heap_begin->distance > row[j])
                {
                    std::pop_heap(heap_begin, heap_end, less);
                    *(heap_end - 1) = distance_pair{row[j], static_cast<std::int32_t>(j)};
                    std::push_heap(heap_begin, heap_end, less);
                }
            }
            std::sort(heap_begin, heap_end, less);
        }
    }

    std::vector<distance_pair> finish() override { return result_; }

private:
    std::vector<float> matrix_;
    std::vector<distance_pair> result_;
};

// ---------------------------------------------------------------------------------------------
// bits (reference: src/topk/singlepass/bits_knn.cu:29-186)
// ---------------------------------------------------------------------------------------------

class bits_knn : public device_knn
{
public:
    explicit bits_knn(bool prefetch) : prefetch_(prefetch) {}
    std::string id() const override { return prefetch_ ? "bits-prefetch" : "bits"; }

    void selection() override
    {
        BITSKNN_CHECK(bitsknn_topk_bits_f32(
            in_dist_gpu(), point_count(), nullptr, 0, nullptr, query_count(), point_count(),
            out_dist_.data(), out_label_.data(), k(), static_cast<std::uint32_t>(k()),
            static_cast<std::uint32_t>(args_.selection_block_size),
            static_cast<std::uint32_t>(args_.items_per_thread[0]), prefetch_ ? 1 : 0, nullptr));
        sync_default_stream();
    }

private:
    bool prefetch_;
};

// `partial-bitonic-regs`: sort-and-merge in registers without a filter
// (reference: src/topk/singlepass/partial_bitonic.cu:217-294, 341-358)
class partial_bitonic_regs : public device_knn
{
public:
    std::string id() const override { return "partial-bitonic-regs"; }

    void selection() override
    {
        BITSKNN_CHECK(bitsknn_topk_partial_bitonic_f32(
            in_dist_gpu(), point_count(), query_count(), point_count(), out_dist_.data(),
            out_label_.data(), k(), static_cast<std::uint32_t>(k()),
            static_cast<std::uint32_t>(args_.selection_block_size), nullptr));
        sync_default_stream();
    }
};

// `bits-sq`: every row is cut into --deg parts that are selected independently (labels shifted
// by the part offset), then the deg*k partial results of a row are selected again with their
// labels (reference: single_query_bits, src/topk/singlepass/bits_knn.cu:116-186).
class single_query_bits : public device_knn
{
public:
    std::string id() const override { return "bits-sq"; }

    void initialize(const knn_args& args) override
    {
        device_knn::initialize(args);
        if (args_.deg > 1)
        {
            if (point_count() % args_.deg != 0)
            {
                throw std::runtime_error("bits-sq: the number of objects must be a multiple of --deg");
            }
            const std::size_t parts = query_count() * args_.deg;
            tmp_dist_ = device_buffer<float>{parts * k()};
            tmp_label_ = device_buffer<std::int32_t>{parts * k()};
            // one counter per row, zero between calls
            counters_ = device_buffer<std::int32_t>{query_count()};
            HIP_CHECK(hipMemsetAsync(counters_.data(), 0, query_count() * sizeof(std::int32_t), nullptr));
            sync_default_stream();
        }
    }

    void selection() override
    {
        BITSKNN_CHECK(bitsknn_topk_bits_parts_f32(
            in_dist_gpu(), query_count(), point_count(), static_cast<std::uint32_t>(std::max<std::size_t>(args_.deg, 1)),
            tmp_dist_.data(), tmp_label_.data(), counters_.data(), out_dist_.data(), out_label_.data(), k(),
            static_cast<std::uint32_t>(k()), static_cast<std::uint32_t>(args_.selection_block_size),
            static_cast<std::uint32_t>(args_.items_per_thread[0]), nullptr));
        sync_default_stream();
    }

private:
    device_buffer<float> tmp_dist_;
    device_buffer<std::int32_t> tmp_label_;
    device_buffer<std::int32_t> counters_;
};

// ---------------------------------------------------------------------------------------------
// bits-fused (reference: src/topk/singlepass/fused_cache_knn.cu:149-216)
// ---------------------------------------------------------------------------------------------

class fused_cache_knn : public device_knn
{
public:
    // arithmetic: BITSKNN_FUSED_EXACT (the reference's id: its arithmetic), BITSKNN_FUSED_FP32 or
    // BITSKNN_FUSED_BF16X3
    explicit fused_cache_knn(int arithmetic = BITSKNN_FUSED_EXACT) : arithmetic_(arithmetic) {}

    std::string id() const override
    {
        return arithmetic_ == BITSKNN_FUSED_BF16X3 ? "fused-cache-bf16x3"
               : arithmetic_ == BITSKNN_FUSED_FP32 ? "fused-cache-mfma"
                                                   : "fused-cache";
    }

    void initialize(const knn_args& args) override
    {
        // no distance matrix is allocated: the kernel never materialises it
        args_ = args;
        args_.dist_layout = matrix_layout::row_major;
        allocate_outputs();
        const auto points = to_dim_major(args_.points, point_count(), dim(), args_.points_layout);
        const auto queries = to_dim_major(args_.queries, query_count(), dim(), args_.queries_layout);
        points_ = device_buffer<float>{points.size()};
        queries_ = device_buffer<float>{queries.size()};
        // BITSKNN_FUSED_TUNING="ranges=R,first_radius=F[,image=I]" in the environment: the launch
        // parameters a tuning sweep varies here (bitsknn_fused_tuning), in place of the library's own
        // choice
        tuned_ = false;
        tuning_ = bitsknn_fused_tuning{};
        if (const char* text = std::getenv("BITSKNN_FUSED_TUNING"); text != nullptr && *text != '\0')
        {
            int ranges = 0;
            int first_radius = 0;
            int image = 0;
            if (std::sscanf(text, "ranges=%d,first_radius=%d,image=%d", &ranges, &first_radius, &image) < 2)
            {
                throw std::runtime_error("BITSKNN_FUSED_TUNING must read ranges=R,first_radius=F[,image=I]");
            }
            tuning_.ranges = ranges;
            tuning_.first_radius = first_radius;
            tuning_.image = image;
            tuned_ = true;
        }
        // partial lists of the point ranges when the queries alone do not fill the GPU (room for the
        // 64 ranges a tuning may ask for), then, from the next multiple of 256 bytes on, room for the
        // stages of the exact arithmetic cut once per call
        const std::size_t lists =
            tuned_ ? query_count() * 64 * k() * 8
                   : bitsknn_fused_workspace_bytes(static_cast<std::int32_t>(query_count()),
                                                   static_cast<std::int32_t>(point_count()), static_cast<int>(k()));
        const std::size_t image =
            arithmetic_ == BITSKNN_FUSED_EXACT
                ? bitsknn_fused_image_bytes(static_cast<int>(dim()), static_cast<std::int32_t>(point_count()))
                : 0;
        workspace_ = device_buffer<unsigned char>{(lists + 255) / 256 * 256 + image};
        transfer_in_.start();
        points_.upload(points.data(), points.size());
        queries_.upload(queries.data(), queries.size());
        sync_default_stream();
        transfer_in_.stop();
    }

    void distances() override {}

    void selection() override
    {
        if (tuned_)
        {
            // the reference's parameters are validated with its messages (no queries: nothing runs),
            // then the launch parameters of this implementation are the ones from the environment
            BITSKNN_CHECK(bitsknn_fused_l2_topk_f32_ex(
                queries_.data(), points_.data(), static_cast<int>(dim()), 0, static_cast<std::int32_t>(point_count()),
                out_dist_.data(), out_label_.data(), static_cast<int>(k()), static_cast<int>(args_.items_per_thread[0]),
                static_cast<int>(args_.items_per_thread[1]), static_cast<int>(args_.items_per_thread[2]),
                static_cast<int>(args_.selection_block_size), static_cast<int>(args_.deg), arithmetic_, nullptr, 0,
                nullptr));
            BITSKNN_CHECK(bitsknn_fused_l2_topk_f32_tuned(
                queries_.data(), points_.data(), static_cast<int>(dim()), static_cast<std::int32_t>(query_count()),
                static_cast<std::int32_t>(point_count()), out_dist_.data(), out_label_.data(), static_cast<int>(k()),
                arithmetic_, &tuning_, workspace_.size() != 0 ? workspace_.data() : nullptr, workspace_.size(),
                nullptr));
        }
        else
        {
            BITSKNN_CHECK(bitsknn_fused_l2_topk_f32_ex(
                queries_.data(), points_.data(), static_cast<int>(dim()), static_cast<std::int32_t>(query_count()),
                static_cast<std::int32_t>(point_count()), out_dist_.data(), out_label_.data(),
                static_cast<int>(k()), static_cast<int>(args_.items_per_thread[0]),
                static_cast<int>(args_.items_per_thread[1]), static_cast<int>(args_.items_per_thread[2]),
                static_cast<int>(args_.selection_block_size), static_cast<int>(args_.deg), arithmetic_,
                workspace_.size() != 0 ? workspace_.data() : nullptr, workspace_.size(), nullptr));
        }
        // synchronises, and fails if a wave of the kernel gave up a wait for a stage
        BITSKNN_CHECK(bitsknn_fused_status(nullptr));
    }

    float transfer_in_seconds() const override { return transfer_in_.seconds(); }

private:
    int arithmetic_;
    bool tuned_ = false;
    bitsknn_fused_tuning tuning_{};
    device_buffer<float> points_;
    device_buffer<float> queries_;
    device_buffer<unsigned char> workspace_;
    knn_host::transfer_timer transfer_in_;
};

// `fused-cache-2pass` (no counterpart among the reference's ids; the same two phases as its runs
// of bits-prefetch next to fused-cache, scripts/run-fused.sh): the partial distances
// ||p||^2 - 2 q.p go to a q x n matrix in the `distances` phase (matrix instructions) and the bits
// kernel selects from it in the `selection` phase.  Unlike the fused kernel its time does not grow
// with k, at the price of the matrix.
class two_pass_knn : public device_knn
{
public:
    std::string id() const override { return "fused-cache-2pass"; }

    void initialize(const knn_args& args) override
    {
        set_dist_impl(make_partial_l2_distance());
        device_knn::initialize(args);
    }

    void selection() override
    {
        BITSKNN_CHECK(bitsknn_topk_bits_f32(
            in_dist_gpu(), point_count(), nullptr, 0, nullptr, query_count(), point_count(),
            out_dist_.data(), out_label_.data(), k(), static_cast<std::uint32_t>(k()), 512, 3, 0, nullptr));
        sync_default_stream();
    }
};

// ---------------------------------------------------------------------------------------------
// distance-only runs (reference: include/bits/distance/dist_runner.hpp:8-15)
// ---------------------------------------------------------------------------------------------

class dist_runner : public device_knn
{
public:
    using factory = std::unique_ptr<device_distance> (*)();
    dist_runner(std::string id, factory make) : id_(std::move(id)), make_(make) {}
    std::string id() const override { return id_; }

    void initialize(const knn_args& args) override
    {
        set_dist_impl(make_());
        device_knn::initialize(args);
        BITSKNN_CHECK(bitsknn_fill_f32(out_dist_.data(), out_dist_.size(), 0.0F, nullptr));
        HIP_CHECK(hipMemsetAsync(out_label_.data(), 0, out_label_.size() * sizeof(std::int32_t), nullptr));
        sync_default_stream();
    }

private:
    std::string id_;
    factory make_;
};

} // namespace

std::vector<std::unique_ptr<knn>> make_algorithms()
{
    std::vector<std::unique_ptr<knn>> algorithms;
    algorithms.push_back(std::make_unique<serial_knn>());
    algorithms.push_back(std::make_unique<parallel_knn>());
    algorithms.push_back(std::make_unique<bits_knn>(false));
    algorithms.push_back(std::make_unique<bits_knn>(true));
    algorithms.push_back(std::make_unique<single_query_bits>());
    algorithms.push_back(std::make_unique<partial_bitonic_regs>());
    algorithms.push_back(std::make_unique<fused_cache_knn>(BITSKNN_FUSED_EXACT));
    algorithms.push_back(std::make_unique<fused_cache_knn>(BITSKNN_FUSED_FP32));
    algorithms.push_back(std::make_unique<fused_cache_knn>(BITSKNN_FUSED_BF16X3));
    algorithms.push_back(std::make_unique<two_pass_knn>());
    algorithms.push_back(std::make_unique<dist_runner>("cublas-dist", &make_expanded_distance));
    algorithms.push_back(std::make_unique<dist_runner>("magma-dist", &make_l2_distance));
    algorithms.push_back(std::make_unique<dist_runner>("magma-part-dist", &make_partial_l2_distance));
    algorithms.push_back(
        std::make_unique<dist_runner>("magma-part-dist-bf16x3", &make_partial_l2_bf16x3_distance));
    return algorithms;
}
