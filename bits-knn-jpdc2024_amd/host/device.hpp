// HIP RAII helpers of the `knn` driver: device buffers, the default stream, event timers and
// error checking.  Counterpart of the reference's cuda_array / cuda_ptr / cuda_stream /
// cuda_event / CUCH helpers (include/bits/cuda_array.hpp:21-132, cuda_stream.hpp:15-202,
// cuda_event.hpp:10-73, cuch.hpp:9-19).
#ifndef KNN_HOST_DEVICE_HPP_
#define KNN_HOST_DEVICE_HPP_

#include <hip/hip_runtime.h>

#include <cstddef>
#include <iostream>
#include <stdexcept>
#include <utility>

#include "bitsknn.h"

// Prints `file:line name: description` and throws, like the reference's CUCH macro.
#define HIP_CHECK(expr) ::knn_host::check_hip((expr), __FILE__, __LINE__)
// Turns a non-zero status of the C ABI into the exception the reference wrappers throw.
#define BITSKNN_CHECK(expr) ::knn_host::check_abi((expr))

namespace knn_host
{

inline void check_hip(hipError_t status, const char* file, int line)
{
    if (status != hipSuccess)
    {
        std::cerr << file << ":" << line << " " << hipGetErrorName(status) << ": "
                  << hipGetErrorString(status) << '\n';
        throw std::runtime_error("HIP error.");
    }
}

inline void check_abi(int status)
{
    if (status != BITSKNN_OK)
    {
        throw std::runtime_error(bitsknn_last_error());
    }
}

// Owning device allocation of `count` elements.
template <typename T>
class device_buffer
{
public:
    device_buffer() = default;
    explicit device_buffer(std::size_t count) : count_(count)
    {
        if (count_ > 0)
        {
            HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&ptr_), count_ * sizeof(T)));
        }
    }
    device_buffer(const device_buffer&) = delete;
    device_buffer& operator=(const device_buffer&) = delete;
    device_buffer(device_buffer&& other) noexcept { swap(other); }
    device_buffer& operator=(device_buffer&& other) noexcept
    {
        if (this != &other)
        {
            release();
            swap(other);
        }
        return *this;
    }
    ~device_buffer() { release(); }

    void release()
    {
        if (ptr_ != nullptr)
        {
            (void)hipFree(ptr_);
        }
        ptr_ = nullptr;
        count_ = 0;
    }

    T* data() const { return ptr_; }
    std::size_t size() const { return count_; }

    void upload(const T* host, std::size_t count)
    {
        HIP_CHECK(hipMemcpyAsync(ptr_, host, count * sizeof(T), hipMemcpyHostToDevice, nullptr));
    }
    void download(T* host, std::size_t count) const
    {
        HIP_CHECK(hipMemcpyAsync(host, ptr_, count * sizeof(T), hipMemcpyDeviceToHost, nullptr));
    }

private:
    void swap(device_buffer& other)
    {
        std::swap(ptr_, other.ptr_);
        std::swap(count_, other.count_);
    }

    T* ptr_ = nullptr;
    std::size_t count_ = 0;
};

// Everything runs on the default stream; a phase ends when the stream is idle.
inline void sync_default_stream() { HIP_CHECK(hipStreamSynchronize(nullptr)); }

// Pair of events around a transfer; seconds() is valid after stop().  The events are created on
// first use so that building the algorithm registry does not touch the device.
class transfer_timer
{
public:
    transfer_timer() = default;
    transfer_timer(const transfer_timer&) = delete;
    transfer_timer& operator=(const transfer_timer&) = delete;
    ~transfer_timer()
    {
        if (begin_ != nullptr)
        {
            (void)hipEventDestroy(begin_);
            (void)hipEventDestroy(end_);
        }
    }
    void start()
    {
        if (begin_ == nullptr)
        {
            HIP_CHECK(hipEventCreate(&begin_));
            HIP_CHECK(hipEventCreate(&end_));
        }
        HIP_CHECK(hipEventRecord(begin_, nullptr));
    }
    void stop()
    {
        HIP_CHECK(hipEventRecord(end_, nullptr));
        HIP_CHECK(hipEventSynchronize(end_));
        recorded_ = true;
    }
    float seconds() const
    {
        if (!recorded_)
        {
            return 0;
        }
        float ms = 0;
        HIP_CHECK(hipEventElapsedTime(&ms, begin_, end_));
        return ms / 1000.0F;
    }

private:
    hipEvent_t begin_ = nullptr;
    hipEvent_t end_ = nullptr;
    bool recorded_ = false;
};

} // namespace knn_host

#endif // KNN_HOST_DEVICE_HPP_
