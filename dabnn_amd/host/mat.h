// bnn::Mat: an NHWC tensor in DEVICE memory (the reference's Mat, dabnn/mat.h:37-155,
// re-hosted on the GPU and given a real batch dimension).
//
//   Float: fp32 [n][h][w][c]
//   Bit:   uint64 [n][h][w][c] where c counts 64-bit words and elem_c the channels
//
// Rows are contiguous (the reference pads rows to 16 bytes and asserts that
// w*c*elemsize is already a multiple of 16, dabnn/mat.h:246, so its layout is
// contiguous too).  Constructor arguments are (h, w, c) in the order every
// caller of the reference passes them.
#pragma once

#include <cstdint>
#include <memory>
#include <string>
#include <vector>

namespace bnn {

enum class DataType { Float, Bit };

class Mat {
   public:
    int n = 1, h = 0, w = 0, c = 0;
    int elem_c = 0;
    DataType data_type = DataType::Float;
    size_t elemsize = 4;
    void *data = nullptr;  // device pointer
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
    bool empty() const { return data == nullptr || total() == 0; }

    void upload(const void *host, size_t nbytes);
    void download(void *host, size_t nbytes) const;
    std::vector<float> to_host_float() const;
    std::vector<uint64_t> to_host_bits() const;

   private:
    size_t data_num_ = 0;
};

}  // namespace bnn
