// Tensor: a host buffer paired with a device buffer, the reference's common/tensor.h:11-40
// with the same members.  cudaStream_t& becomes ko_stream_t& (an opaque stream handle of
// the C ABI).  Three defects of the reference are not carried over: the int-typed
// std::accumulate seed that overflows for large shapes (tensor.h:15), `delete` of a
// `new[]` buffer (tensor.cu:24), and a move assignment that leaks the destination's
// buffers and does not move the size (tensor.cu:13-21).
#ifndef KERNEL_OPTIMIZATION_TENSOR_H
#define KERNEL_OPTIMIZATION_TENSOR_H

#include <cstddef>
#include <functional>
#include <numeric>
#include <vector>

#include "../../ko.h"

class Tensor {
public:
    Tensor(size_t _size_in_bytes);
    Tensor(std::vector<size_t> _shape, size_t byte_per_element)
        : Tensor(byte_per_element *
                 std::accumulate(_shape.begin(), _shape.end(), static_cast<size_t>(1), std::multiplies<size_t>())) {}
    Tensor &operator=(Tensor &&rhs);
    Tensor(Tensor &&rhs);
    Tensor(const Tensor &) = delete;
    Tensor &operator=(const Tensor &) = delete;

    template <typename T>
    T *host_ref() {
        return reinterpret_cast<T *>(this->host_ptr);
    }

    template <typename T>
    T *device_ref() {
        return reinterpret_cast<T *>(this->device_ptr);
    }

    size_t size() const { return this->size_in_bytes; }

    void host_to_device();
    void host_to_device_async(ko_stream_t &stream);
    void device_to_host();
    void device_to_host_async(ko_stream_t &stream);

    ~Tensor();

private:
    void release();
    void *host_ptr;
    void *device_ptr;
    size_t size_in_bytes;
};

#endif  // KERNEL_OPTIMIZATION_TENSOR_H
