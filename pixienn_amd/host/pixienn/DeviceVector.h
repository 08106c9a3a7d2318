// Owning device buffer, the counterpart of the engine's device vector
// (reference: PxCudaVectorT, include/PxTensor.h:440-575): RAII allocation, fill, host<->device
// copies and a blocking asVector().  Move-only; copy() is explicit.
#pragma once

#include <cstddef>
#include <initializer_list>
#include <type_traits>
#include <utility>
#include <vector>

#include "Error.h"

namespace px::hip {

template<typename T>
class DeviceVector
{
    static_assert(std::is_same_v<T, float> || std::is_same_v<T, int>, "float and int buffers only");

public:
    using value_type = T;
    using size_type = std::size_t;

    DeviceVector() = default;

    // Filled on `stream` and waited for, so that the vector can be used on any stream (also a non-blocking
    // one, which does not order itself behind the null stream) once the constructor returns.  Pass the stream
    // the vector will live on: waiting for the null stream drains every blocking stream of the device.
    explicit DeviceVector(size_type n, T value = T(), hipStream_t stream = nullptr)
    {
        allocate(n);
        if (n) {
            fill(value, stream);
            PX_HIP_RUNTIME_CHECK(hipStreamSynchronize(stream));
        }
    }

    DeviceVector(const T* begin, const T* end)
    {
        allocate(static_cast<size_type>(end - begin));
        copyHost(begin, size_);
    }

    explicit DeviceVector(const std::vector<T>& host) : DeviceVector(host.data(), host.data() + host.size()) {}

    DeviceVector(std::initializer_list<T> host) : DeviceVector(host.begin(), host.end()) {}

    DeviceVector(const DeviceVector&) = delete;
    DeviceVector& operator=(const DeviceVector&) = delete;

    DeviceVector(DeviceVector&& rhs) noexcept { swap(rhs); }

    DeviceVector& operator=(DeviceVector&& rhs) noexcept
    {
        if (this != &rhs) {
            release();
            swap(rhs);
        }
        return *this;
    }

    ~DeviceVector() { release(); }

    T* data() noexcept { return data_; }
    const T* data() const noexcept { return data_; }
    size_type size() const noexcept { return size_; }
    bool empty() const noexcept { return size_ == 0; }

    // Ordered on `stream` (the null stream by default), like every kernel of the library.
    void fill(T value, hipStream_t stream = nullptr)
    {
        if constexpr (std::is_same_v<T, float>) PX_HIP_CHECK(pxh_fill_f32(data_, size_, value, stream));
        else PX_HIP_CHECK(pxh_fill_i32(data_, size_, value, stream));
    }

    void copy(const DeviceVector& rhs, hipStream_t stream = nullptr)
    {
        PX_CHECK(rhs.size_ == size_, "copy between device vectors of different sizes");
        if (size_ == 0) return;
        PX_HIP_RUNTIME_CHECK(hipMemcpyAsync(data_, rhs.data_, size_ * sizeof(T), hipMemcpyDeviceToDevice, stream));
    }

    // Blocking host -> device copy of n elements.  `stream` is the stream the vector is used on: work
    // queued there may still read the old contents, so it is waited for first (a non-blocking stream
    // does not order itself against the copy).
    void copyHost(const T* host, size_type n, hipStream_t stream = nullptr)
    {
        PX_CHECK(n <= size_, "host source larger than the device vector");
        if (n == 0) return;
        if (stream) PX_HIP_RUNTIME_CHECK(hipStreamSynchronize(stream));
        PX_HIP_RUNTIME_CHECK(hipMemcpy(data_, host, n * sizeof(T), hipMemcpyHostToDevice));
    }

    void copyHost(const std::vector<T>& host, hipStream_t stream = nullptr) { copyHost(host.data(), host.size(), stream); }

    // Device -> device copy of n elements from a raw device pointer, ordered on `stream`.
    void copyDevice(const T* device, size_type n, hipStream_t stream = nullptr)
    {
        PX_CHECK(n <= size_, "device source larger than the device vector");
        if (n == 0) return;
        PX_HIP_RUNTIME_CHECK(hipMemcpyAsync(data_, device, n * sizeof(T), hipMemcpyDeviceToDevice, stream));
    }

    // Blocking device -> host copy.  `stream` is the stream that last wrote the vector: it is waited
    // for first, since the copy itself only orders behind the null stream and blocking streams.
    std::vector<T> asVector(hipStream_t stream = nullptr) const
    {
        std::vector<T> host(size_);
        if (size_) {
            if (stream) PX_HIP_RUNTIME_CHECK(hipStreamSynchronize(stream));
            PX_HIP_RUNTIME_CHECK(hipMemcpy(host.data(), data_, size_ * sizeof(T), hipMemcpyDeviceToHost));
        }
        return host;
    }

    // Frees the buffer now (the destructor does the same).
    void release() noexcept
    {
        if (data_) (void) hipFree(data_);
        data_ = nullptr;
        size_ = 0;
    }

private:
    void allocate(size_type n)
    {
        size_ = n;
        if (n) PX_HIP_RUNTIME_CHECK(hipMalloc(reinterpret_cast<void**>(&data_), n * sizeof(T)));
    }

    void swap(DeviceVector& rhs) noexcept
    {
        std::swap(data_, rhs.data_);
        std::swap(size_, rhs.size_);
    }

    T* data_ = nullptr;
    size_type size_ = 0;
};

using FloatVector = DeviceVector<float>;
using IntVector = DeviceVector<int>;

}   // px::hip
