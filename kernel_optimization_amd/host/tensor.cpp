// Out-of-line part of Tensor: allocation and the four copies, all through the C ABI (no HIP headers).
// The reference's counterpart is common/tensor.cu:8-42.
#include "kernel_optimization/common/tensor.h"

#include <cstdio>
#include <cstdlib>
#include <limits>
#include <utility>

#include "kernel_optimization/common/common.h"

namespace ko_detail {

DeviceBlock::DeviceBlock(size_t bytes) { checkKoErrors(ko_malloc(&ptr_, bytes)); }

DeviceBlock &DeviceBlock::operator=(DeviceBlock &&other) noexcept {
    std::swap(ptr_, other.ptr_);  // the old allocation leaves with `other`
    return *this;
}

DeviceBlock::~DeviceBlock() {
    if (ptr_ != nullptr) checkKoErrors(ko_free(ptr_));
}

size_t checked_byte_count(const std::vector<size_t> &shape, size_t bytes_per_element) {
    size_t total = bytes_per_element;
    for (size_t extent : shape) {
        if (extent != 0 && total > std::numeric_limits<size_t>::max() / extent) {
            std::fprintf(stderr, "Tensor: shape does not fit size_t\n");
            std::exit(EXIT_FAILURE);
        }
        total *= extent;
    }
    return total;
}

}  // namespace ko_detail

Tensor::Tensor(size_t bytes) : host_(new unsigned char[bytes > 0 ? bytes : 1]), device_(bytes), bytes_(bytes) {}

void Tensor::host_to_device() { checkKoErrors(ko_memcpy_h2d(device_.get(), host_.get(), bytes_)); }

void Tensor::device_to_host() { checkKoErrors(ko_memcpy_d2h(host_.get(), device_.get(), bytes_)); }

void Tensor::host_to_device_async(ko_stream_t &stream) {
    checkKoErrors(ko_memcpy_h2d_async(device_.get(), host_.get(), bytes_, stream));
}

void Tensor::device_to_host_async(ko_stream_t &stream) {
    checkKoErrors(ko_memcpy_d2h_async(host_.get(), device_.get(), bytes_, stream));
}
