#include "mat.h"

#include <hip/hip_runtime_api.h>

#include <stdexcept>

namespace bnn {

static void hip_check(hipError_t e, const char *what) {
    if (e != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}

Mat::Mat(int n_, int h_, int w_, int c_, DataType type, const std::string &name_)
    : n(n_), h(h_), w(w_), data_type(type), name(name_) {
    if (type == DataType::Bit) {
        if (c_ % 64 != 0) throw std::runtime_error("Bit Mat needs a channel count that is a multiple of 64, got " + std::to_string(c_));
        elem_c = c_;
        c = c_ / 64;
        elemsize = 8;
    } else {
        elem_c = c = c_;
        elemsize = 4;
    }
    if (bytes() > 0) hip_check(hipMalloc(&data, bytes()), "hipMalloc");
}

Mat::Mat(size_t len, DataType type, const std::string &name_) : n(1), h(1), w(1), data_type(type), name(name_) {
    c = (int)len;
    elem_c = type == DataType::Bit ? (int)len * 64 : (int)len;
    elemsize = type == DataType::Bit ? 8 : 4;
    data_num_ = len;
    if (bytes() > 0) hip_check(hipMalloc(&data, bytes()), "hipMalloc");
}

Mat::Mat(int n_, int h_, int w_, int c_, void *device_data, DataType type, size_t data_num)
    : n(n_), h(h_), w(w_), data_type(type), data(device_data), external_memory(true), data_num_(data_num) {
    if (type == DataType::Bit) {
        elem_c = c_;
        c = c_ / 64;
        elemsize = 8;
    } else {
        elem_c = c = c_;
        elemsize = 4;
    }
}

Mat::~Mat() {
    if (data && !external_memory) (void)hipFree(data);
}

void Mat::upload(const void *host, size_t nbytes) {
    if (nbytes > bytes()) throw std::runtime_error("Mat::upload: source larger than the tensor");
    hip_check(hipMemcpy(data, host, nbytes, hipMemcpyHostToDevice), "hipMemcpy H2D");
}

void Mat::download(void *host, size_t nbytes) const {
    if (nbytes > bytes()) throw std::runtime_error("Mat::download: destination larger than the tensor");
    hip_check(hipMemcpy(host, data, nbytes, hipMemcpyDeviceToHost), "hipMemcpy D2H");
}

std::vector<float> Mat::to_host_float() const {
    if (data_type != DataType::Float) throw std::runtime_error("to_host_float on a Bit Mat");
    std::vector<float> out(total());
    if (!out.empty()) download(out.data(), bytes());
    return out;
}

std::vector<uint64_t> Mat::to_host_bits() const {
    if (data_type != DataType::Bit) throw std::runtime_error("to_host_bits on a Float Mat");
    std::vector<uint64_t> out(total());
    if (!out.empty()) download(out.data(), bytes());
    return out;
}

}  // namespace bnn
