#include "mat.h"

#include <hip/hip_runtime_api.h>

#include <cmath>
#include <fstream>
#include <ostream>
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
    if (bytes() > 0) hip_check(hipMalloc(&dev, bytes()), "hipMalloc");
}

Mat::Mat(size_t len, DataType type, const std::string &name_) : n(1), h(1), w(1), data_type(type), name(name_) {
    c = (int)len;
    elem_c = type == DataType::Bit ? (int)len * 64 : (int)len;
    elemsize = type == DataType::Bit ? 8 : 4;
    data_num_ = len;
    if (bytes() > 0) hip_check(hipMalloc(&dev, bytes()), "hipMalloc");
}

Mat::Mat(int n_, int h_, int w_, int c_, void *device_data, DataType type, size_t data_num)
    : n(n_), h(h_), w(w_), data_type(type), dev(device_data), external_memory(true), data_num_(data_num) {
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
    if (dev && !external_memory) (void)hipFree(dev);
}

// Copies between host and device go over one stream of their own that does not synchronise with the null stream, and
// wait for it.  A plain hipMemcpy works on the null stream, and a null-stream operation issued by one thread while
// another thread's Net captures its HIP graph fails and invalidates that capture.
static hipStream_t copy_stream() {
    static hipStream_t s = [] {
        hipStream_t created = nullptr;
        hip_check(hipStreamCreateWithFlags(&created, hipStreamNonBlocking), "hipStreamCreate");
        return created;
    }();
    return s;
}

void Mat::upload(const void *host, size_t nbytes) {
    if (nbytes > bytes()) throw std::runtime_error("Mat::upload: source larger than the tensor");
    hip_check(hipMemcpyAsync(dev, host, nbytes, hipMemcpyHostToDevice, copy_stream()), "hipMemcpyAsync H2D");
    hip_check(hipStreamSynchronize(copy_stream()), "hipStreamSynchronize");
    host_valid_ = false;
}

void Mat::download(void *host, size_t nbytes) const {
    if (nbytes > bytes()) throw std::runtime_error("Mat::download: destination larger than the tensor");
    hip_check(hipMemcpyAsync(host, dev, nbytes, hipMemcpyDeviceToHost, copy_stream()), "hipMemcpyAsync D2H");
    hip_check(hipStreamSynchronize(copy_stream()), "hipStreamSynchronize");
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

void Mat::sync_to_host() const {
    if (host_valid_) return;
    if (host_.size() != bytes()) {
        host_.resize(bytes());
        data = host_.empty() ? nullptr : host_.data();
    }
    // the copy does not wait for work queued on other streams; a Net synchronises its own stream at the end of run()
    if (!host_.empty()) download(host_.data(), host_.size());
    host_valid_ = true;
}

bool Mat::operator==(const Mat &m) const {
    if (this == &m || (dev != nullptr && dev == m.dev)) return true;
    if (!(elemsize == m.elemsize && n == m.n && w == m.w && h == m.h && c == m.c && data_type == m.data_type &&
          total() == m.total()))
        return false;
    sync_to_host();
    m.sync_to_host();
    if (data_type == DataType::Float) {
        const float *a = static_cast<const float *>(data), *b = static_cast<const float *>(m.data);
        for (size_t i = 0; i < total(); ++i) {
            if (std::isnan(a[i]) != std::isnan(b[i])) return false;
            if (std::abs(a[i] - b[i]) > 1e-5) return false;
        }
    } else {
        const uint64_t *a = static_cast<const uint64_t *>(data), *b = static_cast<const uint64_t *>(m.data);
        for (size_t i = 0; i < total(); ++i)
            if (a[i] != b[i]) return false;
    }
    return true;
}

void Mat::dump(const std::string &filename) const {
    if (data_type != DataType::Float) throw std::runtime_error("dump writes float Mats");
    std::ofstream ofs(filename);
    for (size_t i = 0; i < total(); ++i) ofs << (*this)[(int)i] << std::endl;
}

std::ostream &operator<<(std::ostream &os, const Mat &mat) {
    os << "n: " << mat.n << ", width: " << mat.w << ", height: " << mat.h << ", channels: " << mat.c << std::endl;
    mat.sync_to_host();
    const size_t shown = mat.total() < 10 ? mat.total() : 10;
    for (size_t i = 0; i < shown; ++i) {
        if (mat.data_type == DataType::Float)
            os << static_cast<const float *>(mat.data)[i] << ", ";
        else
            os << std::hex << static_cast<const uint64_t *>(mat.data)[i] << std::dec << ", ";
    }
    return os;
}

}  // namespace bnn
