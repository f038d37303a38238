// Tensor: one host buffer and one device buffer of the same size, with copies in both directions.
// Public interface of the reference's class (common/tensor.h:11-40): construction from a byte count or
// from a shape and an element size, host_ref<T>() / device_ref<T>(), the four copy methods (the
// asynchronous ones take the stream by reference; here an opaque ko_stream_t of the C ABI), move
// assignment, no copying.  The inside is different: both buffers are owned by small RAII holders, so
// moves are member-wise and cannot leak, the element count is formed in size_t with an overflow check
// (the reference seeds std::accumulate with an int, tensor.h:15), and the host array is released with the
// form of delete that matches its allocation (the reference mixes new[] and delete, tensor.cu:24).
#ifndef KERNEL_OPTIMIZATION_TENSOR_H
#define KERNEL_OPTIMIZATION_TENSOR_H

#include <cstddef>
#include <memory>
#include <vector>

#include "../../ko.h"

namespace ko_detail {

// Device allocation of the C ABI, freed on destruction.
class DeviceBlock {
public:
    DeviceBlock() = default;
    explicit DeviceBlock(size_t bytes);
    DeviceBlock(DeviceBlock &&other) noexcept : ptr_(other.ptr_) { other.ptr_ = nullptr; }
    DeviceBlock &operator=(DeviceBlock &&other) noexcept;
    DeviceBlock(const DeviceBlock &) = delete;
    DeviceBlock &operator=(const DeviceBlock &) = delete;
    ~DeviceBlock();
    void *get() const { return ptr_; }

private:
    void *ptr_ = nullptr;
};

// bytes_per_element * product(shape), or an abort with a message if that does not fit size_t.
size_t checked_byte_count(const std::vector<size_t> &shape, size_t bytes_per_element);

}  // namespace ko_detail

class Tensor {
public:
    explicit Tensor(size_t bytes);
    Tensor(std::vector<size_t> shape, size_t bytes_per_element)
        : Tensor(ko_detail::checked_byte_count(shape, bytes_per_element)) {}

    Tensor(Tensor &&) noexcept = default;
    Tensor &operator=(Tensor &&) noexcept = default;  // the destination's old buffers are released
    Tensor(const Tensor &) = delete;
    Tensor &operator=(const Tensor &) = delete;
    ~Tensor() = default;

    template <typename T>
    T *host_ref() {
        return reinterpret_cast<T *>(host_.get());
    }
    template <typename T>
    T *device_ref() {
        return static_cast<T *>(device_.get());
    }
    size_t size() const { return host_ ? bytes_ : 0; }

    void host_to_device();
    void host_to_device_async(ko_stream_t &stream);
    void device_to_host();
    void device_to_host_async(ko_stream_t &stream);

private:
    std::unique_ptr<unsigned char[]> host_;
    ko_detail::DeviceBlock device_;
    size_t bytes_ = 0;
};

#endif  // KERNEL_OPTIMIZATION_TENSOR_H
