// bnn::Mat: an NHWC tensor (the reference's Mat, dabnn/mat.h:37-155) whose working copy lives in DEVICE memory and
// which has a real batch dimension.
//
//   Float: fp32 [n][h][w][c]
//   Bit:   uint64 [n][h][w][c] where c counts 64-bit words and elem_c the channels
//
// Rows are contiguous (the reference pads rows to 16 bytes and asserts that w*c*elemsize is already a multiple of
// 16, dabnn/mat.h:246, so its layout is contiguous too).  Constructor arguments are (h, w, c) in the order every
// caller of the reference passes them.
//
// Host access as in the reference: `data`, `operator T *`, `operator[]`, `operator==`, `point<T>`, `dump` and `<<`
// work on a host mirror of the device memory.  The mirror is filled on demand -- by Net::get_blob, which every
// reference caller goes through, and by each of the accessors -- and marked stale whenever kernels may have written
// the device copy (Net::run); a Mat obtained before a run shows that run's values after the next get_blob or
// accessor call on it.  The mirror is a read-only view: writes through it do not reach the device (the reference's
// callers only read blobs; inputs go through Net::run).  `dev` is the device pointer the kernels work on.
#pragma once

#include <cstdint>
#include <iosfwd>
#include <memory>
#include <string>
#include <vector>

// The C++ classes are part of the library's surface (bnn::Net / bnn::Mat / the layers, as in the reference), so they
// are exported although the library is built with hidden visibility.
#define BNN_API __attribute__((visibility("default")))

namespace bnn {

enum class DataType { Float, Bit };

class BNN_API Mat {
   public:
    int n = 1, h = 0, w = 0, c = 0;
    int elem_c = 0;
    DataType data_type = DataType::Float;
    size_t elemsize = 4;
    mutable void *data = nullptr;  // host mirror (null until the first get_blob / accessor); see sync_to_host()
    void *dev = nullptr;           // device memory
    bool external_memory = false;
    std::string name;

    Mat() = default;
    // owning; c is the channel count (a multiple of 64 for Bit)
    Mat(int n, int h, int w, int c, DataType type, const std::string &name = "");
    Mat(int h, int w, int c, DataType type, const std::string &name = "") : Mat(1, h, w, c, type, name) {}
    // owning, flat: len elements (floats or words)
    Mat(size_t len, DataType type, const std::string &name = "");
    // borrowed device memory
    Mat(int n, int h, int w, int c, void *device_data, DataType type, size_t data_num = 0);
    ~Mat();
    Mat(const Mat &) = delete;
    Mat &operator=(const Mat &) = delete;

    // element count: words for Bit, floats for Float (data_num_ when given, as dabnn/mat.h:597-603)
    size_t total() const { return data_num_ ? data_num_ : (size_t)n * h * w * c; }
    size_t bytes() const { return total() * elemsize; }
    bool empty() const { return dev == nullptr || total() == 0; }

    void upload(const void *host, size_t nbytes);
    void download(void *host, size_t nbytes) const;
    std::vector<float> to_host_float() const;
    std::vector<uint64_t> to_host_bits() const;

    // Brings the host mirror up to date with the device copy (allocates it on first use); waits for the device.
    void sync_to_host() const;
    // The device copy may have changed: the next host access copies it again.
    void mark_device_written() const { host_valid_ = false; }

    // the reference's host accessors (dabnn/mat.h:72,94,101-116)
    template <typename T>
    operator T *() {
        sync_to_host();
        return static_cast<T *>(data);
    }
    template <typename T>
    operator const T *() const {
        sync_to_host();
        return static_cast<const T *>(data);
    }
    const float &operator[](int i) const {
        sync_to_host();
        return static_cast<const float *>(data)[i];
    }
    // Equal shapes and types, floats within 1e-5 of each other with NaN only where the other has NaN, words equal
    // (dabnn/mat.h:295-331; a Bit Mat is compared word by word, which is what the reference means to do).
    bool operator==(const Mat &m) const;
    bool operator!=(const Mat &m) const { return !(*this == m); }
    template <typename T>
    const T *point(int n_, int h_, int w_) const {
        sync_to_host();
        return static_cast<const T *>(data) + (((size_t)n_ * h + h_) * w + w_) * c;
    }
    template <typename T>
    const T *point(int h_, int w_) const {
        return point<T>(0, h_, w_);
    }
    // one element per line (dabnn/mat.h:651-654)
    void dump(const std::string &filename) const;
    friend BNN_API std::ostream &operator<<(std::ostream &os, const Mat &mat);

   private:
    size_t data_num_ = 0;
    mutable std::vector<unsigned char> host_;
    mutable bool host_valid_ = false;
};

}  // namespace bnn
