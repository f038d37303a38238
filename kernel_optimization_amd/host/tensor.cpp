// Tensor over the C ABI (reference: common/tensor.cu:8-42).  Plain C++: no HIP headers.
#include "kernel_optimization/common/tensor.h"
#include "kernel_optimization/common/common.h"

#include <cstdint>

Tensor::Tensor(size_t _size_in_bytes) : host_ptr(nullptr), device_ptr(nullptr), size_in_bytes(_size_in_bytes) {
    this->host_ptr = new uint8_t[this->size_in_bytes ? this->size_in_bytes : 1];
    checkKoErrors(ko_malloc(&this->device_ptr, this->size_in_bytes));
}

Tensor::Tensor(Tensor &&rhs) : host_ptr(rhs.host_ptr), device_ptr(rhs.device_ptr), size_in_bytes(rhs.size_in_bytes) {
    rhs.host_ptr = nullptr;
    rhs.device_ptr = nullptr;
    rhs.size_in_bytes = 0;
}

Tensor &Tensor::operator=(Tensor &&rhs) {
    if (this != &rhs) {
        this->release();
        this->host_ptr = rhs.host_ptr;
        this->device_ptr = rhs.device_ptr;
        this->size_in_bytes = rhs.size_in_bytes;
        rhs.host_ptr = nullptr;
        rhs.device_ptr = nullptr;
        rhs.size_in_bytes = 0;
    }
    return *this;
}

void Tensor::release() {
    if (this->host_ptr) delete[] reinterpret_cast<uint8_t *>(this->host_ptr);
    if (this->device_ptr) checkKoErrors(ko_free(this->device_ptr));
    this->host_ptr = nullptr;
    this->device_ptr = nullptr;
}

Tensor::~Tensor() { this->release(); }

void Tensor::host_to_device() { checkKoErrors(ko_memcpy_h2d(this->device_ptr, this->host_ptr, this->size_in_bytes)); }

void Tensor::host_to_device_async(ko_stream_t &stream) {
    checkKoErrors(ko_memcpy_h2d_async(this->device_ptr, this->host_ptr, this->size_in_bytes, stream));
}

void Tensor::device_to_host() { checkKoErrors(ko_memcpy_d2h(this->host_ptr, this->device_ptr, this->size_in_bytes)); }

void Tensor::device_to_host_async(ko_stream_t &stream) {
    checkKoErrors(ko_memcpy_d2h_async(this->host_ptr, this->device_ptr, this->size_in_bytes, stream));
}
