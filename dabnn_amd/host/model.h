// A .dab model (common/dab.fbs of the reference) parsed into host structures and checked, without touching the GPU.
//
// parse_model() walks the FlatBuffers tables by vtable slot with every access bounds-checked (std::invalid_argument on
// a buffer that does not hold what its offsets promise).  check_model() then does what Net::prepare of the reference
// does implicitly while it builds layers (dabnn/net.cpp:56-270): shape inference as common/Shaper.cpp, the symmetric
// pads / strides rule, and the size relations between a layer's tensors that the kernels rely on (a weight tensor that
// is shorter than its layer's geometry says would make a kernel read past its allocation), as std::runtime_error.
// bnn::Net builds its device objects from the checked description.
#pragma once

#include <cstddef>
#include <cstdint>
#include <map>
#include <string>
#include <vector>

namespace bnn {

// flatbnn::LayerType (common/dab.fbs)
enum ModelLayerType {
    kFpConv2D = 0, kAvePool, kMaxPool, kRelu, kSoftmax, kFC, kAdd, kConcat, kBinConv2D, kAffine, kBinarize, kSplit, kShuffle, kPRelu,
    kLayerTypeCount
};
const char *layer_type_name(int type);

struct TensorDesc {
    std::string name;
    std::vector<uint32_t> shape;
    bool is_bit = false;
    const void *data = nullptr;  // into the model buffer: uint64 words (bit) or floats
    size_t len = 0;              // elements
    bool align_hwc_to_128 = false;
};

struct InputDesc {
    std::string name;
    std::vector<uint32_t> shape;
};

struct LayerDesc {
    int type = -1;
    std::string name;
    std::vector<std::string> inputs;   // one entry except Add (2) and Concat (n)
    std::vector<std::string> outputs;  // one entry except Split (2)
    std::string weight, bias;          // convolutions
    std::string a, b;                  // Affine
    std::string slope;                 // PRelu
    std::vector<int32_t> pads, strides, dilations, kernel_shape;
    int axis = 0;  // Concat
    // filled by check_model for convolutions and pools
    int pad_h = 0, pad_w = 0, stride_h = 1, stride_w = 1, dil_h = 1, dil_w = 1;
};

struct ModelDesc {
    uint32_t version = 0;
    std::vector<InputDesc> inputs;
    std::vector<TensorDesc> initializers;
    std::vector<LayerDesc> layers;
    // filled by check_model: NHWC shape (N = 1) of every blob, and whether it holds packed words
    std::map<std::string, std::vector<uint32_t>> shapes;
    std::map<std::string, bool> is_bit;
};

constexpr uint32_t kModelVersion = 2;  // BNN_LATEST_MODEL_VERSION, common/macros.h:6

// len = bytes the caller vouches for; pass SIZE_MAX for a buffer of unknown extent (the reference's read_buf(ptr)).
ModelDesc parse_model(const void *buf, size_t len);
void check_model(ModelDesc &model, bool run_fconv);

}  // namespace bnn
