#include "model.h"

#include <set>
#include <sstream>
#include <stdexcept>

#include "flatbuf.h"

namespace bnn {

namespace {

// vtable slots of common/dab.fbs (declaration order)
enum ModelSlot { M_LAYERS = 0, M_INITIALIZERS = 1, M_INPUTS = 2, M_VERSION = 3 };
enum TensorSlot { T_DATA_TYPE = 0, T_BIN_DATA = 1, T_FLOAT_DATA = 2, T_SHAPE = 3, T_NAME = 4, T_ALIGN = 5 };
enum InputSlot { I_SHAPE = 0, I_NAME = 1 };
enum LayerSlot {
    L_TYPE = 0, L_FPCONV = 1, L_BINCONV = 2, L_AVEPOOL = 3, L_MAXPOOL = 4, L_RELU = 5, L_SOFTMAX = 6, L_FC = 7, L_ADD = 8,
    L_CONCAT = 9, L_AFFINE = 10, L_BINARIZE = 11, L_SPLIT = 12, L_SHUFFLE = 13, L_NAME = 14, L_PRELU = 15
};

const char *kLayerTypeNames[kLayerTypeCount] = {"FpConv2D", "AvePool", "MaxPool", "Relu",     "Softmax", "FC",      "Add",
                                                "Concat",   "BinConv2D", "Affine", "Binarize", "Split",   "Shuffle", "PRelu"};

[[noreturn]] void fail(const std::string &msg) { throw std::runtime_error(msg); }
void require(bool cond, const std::string &msg) {
    if (!cond) fail(msg);
}

template <class T>
std::string list_str(const std::vector<T> &v) {
    std::stringstream ss;
    for (size_t i = 0; i < v.size(); ++i) ss << (i ? "," : "") << v[i];
    return ss.str();
}

std::vector<std::string> str_vec(const fb::Table &t, int slot) {
    std::vector<std::string> out;
    const uint32_t n = t.vec_len(slot);
    for (uint32_t i = 0; i < n; ++i) out.push_back(t.vec_str(slot, i));
    return out;
}

// pads / strides arrive with 2 or 4 entries; 4 entries must be symmetric (dabnn/net.cpp:174-185)
void check_symmetric(const std::vector<int32_t> &v, const char *what) {
    require(v.size() == 2 || (v.size() == 4 && v[0] == v[2] && v[1] == v[3]),
            std::string(what) + " must have 2 entries or 4 symmetric ones, got " + list_str(v));
}

// Output extent of a convolution or pooling window (common/Shaper.cpp:34-54,127-145); throws when it is empty.
uint32_t window_out(uint32_t in, int pad, int k, int dil, int stride, const std::string &layer) {
    const int64_t extent = (int64_t)dil * (k - 1) + 1;
    const int64_t span = (int64_t)in + 2 * (int64_t)pad - extent;
    require(span >= 0, "layer " + layer + ": the window is larger than its padded input");
    return (uint32_t)(span / stride + 1);
}

}  // namespace

const char *layer_type_name(int type) { return type >= 0 && type < kLayerTypeCount ? kLayerTypeNames[type] : "unknown"; }

ModelDesc parse_model(const void *buf, size_t len) {
    if (buf == nullptr) throw std::invalid_argument("null model buffer");
    if (len == SIZE_MAX) len = SIZE_MAX - reinterpret_cast<uintptr_t>(buf);  // unknown extent: only wrap-around is refused
    const fb::Table root = fb::root(buf, len);
    ModelDesc m;
    m.version = root.scalar<uint32_t>(M_VERSION, 0);
    // the version comes first, as in the reference (dabnn/net.cpp:56-58): a file of another version is reported as
    // such and not as malformed
    if (m.version != kModelVersion) return m;

    for (uint32_t i = 0; i < root.vec_len(M_INPUTS); ++i) {
        const fb::Table in = root.vec_table(M_INPUTS, i);
        InputDesc d;
        d.shape = in.vec_copy<uint32_t>(I_SHAPE);
        d.name = in.str(I_NAME);
        m.inputs.push_back(d);
    }
    for (uint32_t i = 0; i < root.vec_len(M_INITIALIZERS); ++i) {
        const fb::Table t = root.vec_table(M_INITIALIZERS, i);
        TensorDesc d;
        d.name = t.str(T_NAME);
        d.shape = t.vec_copy<uint32_t>(T_SHAPE);
        d.is_bit = t.scalar<int8_t>(T_DATA_TYPE, 0) == 1;
        d.align_hwc_to_128 = t.scalar<uint8_t>(T_ALIGN, 0) != 0;
        uint32_t n = 0;
        if (d.is_bit)
            d.data = t.vec<uint64_t>(T_BIN_DATA, &n);
        else
            d.data = t.vec<float>(T_FLOAT_DATA, &n);
        d.len = n;
        m.initializers.push_back(d);
    }
    for (uint32_t i = 0; i < root.vec_len(M_LAYERS); ++i) {
        const fb::Table layer = root.vec_table(M_LAYERS, i);
        LayerDesc d;
        d.type = layer.scalar<int8_t>(L_TYPE, 0);
        d.name = layer.str(L_NAME);
        auto param = [&](int slot) {
            const fb::Table p = layer.table(slot);
            if (!p.valid()) fail(std::string(layer_type_name(d.type)) + " layer " + d.name + " without parameters");
            return p;
        };
        switch (d.type) {
            case kFpConv2D:
            case kBinConv2D: {
                const fb::Table p = param(d.type == kFpConv2D ? L_FPCONV : L_BINCONV);
                d.inputs = {p.str(0)};
                d.weight = p.str(1), d.bias = p.str(2);
                d.pads = p.vec_copy<int32_t>(3), d.strides = p.vec_copy<int32_t>(4), d.dilations = p.vec_copy<int32_t>(5);
                d.outputs = {p.str(6)};
                break;
            }
            case kAvePool:
            case kMaxPool: {
                const fb::Table p = param(d.type == kMaxPool ? L_MAXPOOL : L_AVEPOOL);
                d.inputs = {p.str(0)};
                d.kernel_shape = p.vec_copy<int32_t>(1), d.pads = p.vec_copy<int32_t>(2), d.strides = p.vec_copy<int32_t>(3);
                d.outputs = {p.str(4)};
                break;
            }
            case kRelu: {
                const fb::Table p = param(L_RELU);
                d.inputs = {p.str(0)}, d.outputs = {p.str(1)};
                break;
            }
            case kAdd: {
                const fb::Table p = param(L_ADD);
                d.inputs = {p.str(0), p.str(1)}, d.outputs = {p.str(2)};
                break;
            }
            case kConcat: {
                const fb::Table p = param(L_CONCAT);
                d.inputs = str_vec(p, 0);
                d.axis = p.scalar<int32_t>(1, 0);
                d.outputs = {p.str(2)};
                break;
            }
            case kAffine: {
                const fb::Table p = param(L_AFFINE);
                d.inputs = {p.str(0)}, d.a = p.str(1), d.b = p.str(2), d.outputs = {p.str(3)};
                break;
            }
            case kSplit: {
                const fb::Table p = param(L_SPLIT);
                d.inputs = {p.str(0)};
                d.outputs = str_vec(p, 1);
                break;
            }
            case kShuffle: {
                const fb::Table p = param(L_SHUFFLE);
                d.inputs = {p.str(0)}, d.outputs = {p.str(1)};
                break;
            }
            case kPRelu: {
                const fb::Table p = param(L_PRELU);
                d.inputs = {p.str(0)}, d.slope = p.str(1), d.outputs = {p.str(2)};
                break;
            }
            default:
                break;  // reported by check_model as "Not supported op"
        }
        m.layers.push_back(d);
    }
    return m;
}

void check_model(ModelDesc &m, bool run_fconv) {
    require(m.version == kModelVersion, "The model version should be " + std::to_string(kModelVersion) + ", got " +
                                            std::to_string(m.version) + " instead.");
    m.shapes.clear(), m.is_bit.clear();
    require(!m.inputs.empty(), "the model has no input");
    {
        const InputDesc &in = m.inputs[0];  // the first one only (dabnn/net.cpp:59-70)
        require(in.shape.size() == 4, "input shape must be NHWC");
        require(in.shape[1] > 0 && in.shape[2] > 0 && in.shape[3] > 0, "input " + in.name + " has an empty dimension");
        require((uint64_t)in.shape[1] * in.shape[2] * in.shape[3] < (1ull << 31), "input " + in.name + " is too large");
        m.shapes[in.name] = in.shape;
        m.is_bit[in.name] = false;
    }
    std::map<std::string, const TensorDesc *> inits;
    for (const TensorDesc &t : m.initializers) {
        uint64_t want = 1;
        for (uint32_t d : t.shape) {
            require(d > 0, "tensor " + t.name + " has an empty dimension");
            want *= d;
            require(want < (1ull << 40), "tensor " + t.name + " is too large");
        }
        if (t.is_bit) {
            require(t.shape.size() == 4, "bit tensor " + t.name + " must be 4-D");
            require(t.len > 0 && t.len % t.shape[0] == 0, "bit tensor " + t.name + " has a bad length");
            // shape is [n][kh][kw][c]; the word count per filter may include the padding to 128 bits
            // (tools/onnx2bnn/OnnxConverter.cpp:121-156) and never more
            const uint64_t bits = (uint64_t)t.shape[1] * t.shape[2] * t.shape[3];
            const uint64_t per = t.len / t.shape[0];
            require(per * 64 >= bits && per <= (bits + 127) / 128 * 2,
                    "bit tensor " + t.name + " holds " + std::to_string(per) + " words per filter, its shape " +
                        list_str(t.shape) + " needs " + std::to_string((bits + 63) / 64));
        } else {
            require(t.shape.size() == 4 || t.shape.size() == 1, "float tensor " + t.name + " must be 1-D or 4-D");
            require(t.len == want, "float tensor " + t.name + " does not match its shape");
        }
        m.shapes[t.name] = t.shape;
        m.is_bit[t.name] = t.is_bit;
        inits[t.name] = &t;
    }

    auto shape_of = [&](const std::string &n) -> const std::vector<uint32_t> & {
        auto it = m.shapes.find(n);
        if (it == m.shapes.end()) throw std::out_of_range("Key " + n + " not found.");
        return it->second;
    };
    auto blob4 = [&](const std::string &n, const std::string &layer) -> const std::vector<uint32_t> & {
        const auto &s = shape_of(n);
        require(s.size() == 4, "layer " + layer + ": blob " + n + " is not 4-D");
        return s;
    };
    auto init_of = [&](const std::string &n, const std::string &layer) -> const TensorDesc & {
        auto it = inits.find(n);
        if (it == inits.end()) {
            (void)shape_of(n);  // an unknown name is a key error, as in the reference
            fail("layer " + layer + ": " + n + " is not an initializer");
        }
        return *it->second;
    };
    // A layer that makes a new blob must not name it like the input, an initializer, an earlier output or one of the
    // scratch blobs a BinConv registers: Net::prepare would keep the blob that exists, of another size, and the
    // layer's kernel would write its own geometry into it.
    std::set<std::string> scratch_names;
    auto fresh_name = [&](const std::string &n, const std::string &layer) {
        require(m.shapes.find(n) == m.shapes.end() && scratch_names.find(n) == scratch_names.end(),
                "layer " + layer + ": output " + n + " names a blob that already exists");
    };
    auto set_out = [&](const std::string &n, uint32_t h, uint32_t w, uint32_t c, bool bit, const std::string &layer) {
        fresh_name(n, layer);
        // the element count of one image and of the output row index must fit the int fields of Mat and the kernels
        require((uint64_t)h * w * c < (1ull << 31), "layer " + layer + ": output " + n + " is too large");
        m.shapes[n] = {1, h, w, c};
        m.is_bit[n] = bit;
    };
    auto alias = [&](const std::string &out, const std::string &in) {  // ADD_INPLACE_LAYER
        // a second name for the input's blob; re-pointing an existing name (the net's input, say) at another blob
        // would hand its earlier users' sizes to a blob of another size
        if (out != in) fresh_name(out, "(in place) " + in);
        const auto s = shape_of(in);
        const bool bit = m.is_bit[in];
        m.shapes[out] = s;
        m.is_bit[out] = bit;
    };
    auto float_vec = [&](const std::string &n, uint32_t want, const std::string &layer, const char *what) {
        const TensorDesc &t = init_of(n, layer);
        require(!t.is_bit && t.len == want, "layer " + layer + ": " + what + " " + n + " must hold " + std::to_string(want) + " floats");
    };

    for (LayerDesc &l : m.layers) {
        switch (l.type) {
            case kFpConv2D:
            case kBinConv2D: {
                check_symmetric(l.pads, "pads");
                check_symmetric(l.strides, "strides");
                l.pad_h = l.pads[0], l.pad_w = l.pads[1], l.stride_h = l.strides[0], l.stride_w = l.strides[1];
                l.dil_h = l.dilations.size() >= 1 ? l.dilations[0] : 1;
                l.dil_w = l.dilations.size() >= 2 ? l.dilations[1] : l.dil_h;
                require(l.pad_h >= 0 && l.pad_w >= 0 && l.pad_h < (1 << 15) && l.pad_w < (1 << 15), "layer " + l.name + ": bad pads " + list_str(l.pads));
                require(l.stride_h > 0 && l.stride_w > 0, "layer " + l.name + ": strides must be positive, got " + list_str(l.strides));
                require(l.dil_h > 0 && l.dil_w > 0, "layer " + l.name + ": dilations must be positive");
                const auto &is = blob4(l.inputs[0], l.name);
                const TensorDesc &wt = init_of(l.weight, l.name);
                require(wt.shape.size() == 4, "layer " + l.name + ": weight " + l.weight + " must be [cout][kh][kw][cin]");
                const auto &ws = wt.shape;
                require(!m.is_bit[l.inputs[0]], l.type == kBinConv2D ? "BinConv input must be float" : "FloatConv input must be float");
                require(ws[3] == is[3], "layer " + l.name + ": weight " + l.weight + " has " + std::to_string(ws[3]) +
                                            " input channels, the input blob " + std::to_string(is[3]));
                require(ws[1] <= (1u << 15) && ws[2] <= (1u << 15), "layer " + l.name + ": kernel " + std::to_string(ws[1]) + "x" +
                                                                        std::to_string(ws[2]) + " is too large");
                const uint32_t oh = window_out(is[1], l.pad_h, (int)ws[1], l.dil_h, l.stride_h, l.name);
                const uint32_t ow = window_out(is[2], l.pad_w, (int)ws[2], l.dil_w, l.stride_w, l.name);
                if (l.type == kBinConv2D) {
                    require(l.dil_h == 1 && l.dil_w == 1, "BinConv dilation must be 1");
                    require(wt.is_bit, "BinConv weight must be Bit");
                    require(is[3] % 64 == 0, "BinConv needs a multiple of 64 input channels, got " + std::to_string(is[3]));
                    const uint64_t per = wt.len / ws[0], cw = is[3] / 64;
                    // the direct 3x3 kernel walks filters of exactly 9 * C/64 words (dabnn/layers/BinConv.cpp:100-126)
                    if (ws[1] == 3 && ws[2] == 3 && (is[3] == 64 || is[3] == 128 || is[3] == 256 || is[3] == 512))
                        require(per == 9 * cw, "layer " + l.name + ": weight " + l.weight + " holds " + std::to_string(per) +
                                                   " words per filter, a 3x3 filter over " + std::to_string(is[3]) +
                                                   " channels has " + std::to_string(9 * cw));
                } else {
                    require(!wt.is_bit, "FloatConv weight must be float");
                    require(l.dil_h == l.dil_w, "FloatConv needs equal dilations");
                }
                if (!l.bias.empty()) float_vec(l.bias, ws[0], l.name, "bias");
                set_out(l.outputs[0], oh, ow, ws[0], false, l.name);
                if (l.type == kBinConv2D) {
                    // the scratch blobs the layer registers under the reference's names (dabnn/layers/BinConv.cpp:17-57)
                    for (const char *prefix : {"binaized_for_", "col_for_"}) {
                        const std::string scratch = prefix + l.outputs[0] + "_cal";
                        fresh_name(scratch, l.name);
                        scratch_names.insert(scratch);
                    }
                    // the transposed weights are registered too; two layers may share a weight
                    require(m.shapes.find("trans_" + l.weight) == m.shapes.end(),
                            "layer " + l.name + ": trans_" + l.weight + " names a blob that already exists");
                    scratch_names.insert("trans_" + l.weight);
                }
                (void)run_fconv;  // a skipped float convolution still defines its output blob (dabnn/net.cpp:145-170)
                break;
            }
            case kAffine: {
                alias(l.outputs[0], l.inputs[0]);
                const auto &s = blob4(l.inputs[0], l.name);
                require(!m.is_bit[l.inputs[0]], "Affine input must be float");
                float_vec(l.a, s[3], l.name, "coefficient");
                float_vec(l.b, s[3], l.name, "coefficient");
                break;
            }
            case kAdd: {
                require(shape_of(l.inputs[0]) == shape_of(l.inputs[1]), "Add operands differ in size");
                require(!m.is_bit[l.inputs[0]] && !m.is_bit[l.inputs[1]], "Add inputs must be float");
                alias(l.outputs[0], l.inputs[0]);
                break;
            }
            case kRelu:
                (void)shape_of(l.inputs[0]);
                require(!m.is_bit[l.inputs[0]], "Relu input must be float");
                alias(l.outputs[0], l.inputs[0]);
                break;
            case kPRelu: {
                const auto &s = blob4(l.inputs[0], l.name);
                require(!m.is_bit[l.inputs[0]], "PRelu input must be float");
                const TensorDesc &sl = init_of(l.slope, l.name);
                require(!sl.is_bit && (sl.len == 1 || sl.len == s[3]), "slope must have size 1 or input.channels");
                alias(l.outputs[0], l.inputs[0]);
                break;
            }
            case kMaxPool:
            case kAvePool: {
                require(l.kernel_shape.size() == 2 && l.pads.size() >= 2 && l.strides.size() >= 2, "pool layer with malformed attributes");
                require(l.kernel_shape[0] > 0 && l.kernel_shape[1] > 0 && l.strides[0] > 0 && l.strides[1] > 0,
                        "global pooling must be exported with an explicit kernel and stride");
                require(l.pads[0] >= 0 && l.pads[1] >= 0 && l.pads[0] < (1 << 15) && l.pads[1] < (1 << 15), "layer " + l.name + ": bad pads " + list_str(l.pads));
                l.pad_h = l.pads[0], l.pad_w = l.pads[1], l.stride_h = l.strides[0], l.stride_w = l.strides[1];
                const auto &is = blob4(l.inputs[0], l.name);
                require(!m.is_bit[l.inputs[0]], "pooling input must be float");
                const uint32_t oh = window_out(is[1], l.pad_h, l.kernel_shape[0], 1, l.stride_h, l.name);  // common/Shaper.cpp:127-145
                const uint32_t ow = window_out(is[2], l.pad_w, l.kernel_shape[1], 1, l.stride_w, l.name);
                require(l.kernel_shape[0] <= (1 << 15) && l.kernel_shape[1] <= (1 << 15), "layer " + l.name + ": pooling window is too large");
                set_out(l.outputs[0], oh, ow, is[3], false, l.name);
                break;
            }
            case kConcat: {  // dabnn/net.cpp:230-236: two inputs, channel axis; shape as common/Shaper.cpp:157-178
                require(l.axis == 3, "Concat: axis must be 3");
                require(l.inputs.size() == 2, "Concat takes two inputs");
                const auto &s1 = blob4(l.inputs[0], l.name);
                const auto &s2 = blob4(l.inputs[1], l.name);
                require(s1[1] == s2[1] && s1[2] == s2[2], "Wrong input for concat");
                require(!m.is_bit[l.inputs[0]] && !m.is_bit[l.inputs[1]], "Concat inputs must be float");
                set_out(l.outputs[0], s1[1], s1[2], s1[3] + s2[3], false, l.name);
                break;
            }
            case kSplit: {  // dabnn/net.cpp:245-250, dabnn/layers/Split.h:16-24; shape as common/Shaper.cpp:245-260
                const auto s = blob4(l.inputs[0], l.name);
                require(l.outputs.size() == 2, "Split makes two outputs");
                require(m.is_bit[l.inputs[0]], "Split only supports bit mat");
                require(s[3] % 128 == 0 && s[3] <= 512, "Split: " + std::to_string(s[3]) + " channels");
                for (const std::string &o : l.outputs) {
                    fresh_name(o, l.name);
                    m.shapes[o] = {s[0], s[1], s[2], s[3] / 2};
                    m.is_bit[o] = true;
                }
                break;
            }
            case kShuffle: {  // dabnn/net.cpp:251-256, dabnn/layers/Shuffle.h:14-21
                const auto &s = blob4(l.inputs[0], l.name);
                require(m.is_bit[l.inputs[0]], "Shuffle only supports bit mat");
                require(s[3] % 128 == 0 && s[3] <= 512, "Shuffle: " + std::to_string(s[3]) + " channels");
                alias(l.outputs[0], l.inputs[0]);
                break;
            }
            default:
                fail(std::string("Not supported op ") + layer_type_name(l.type));
        }
    }
}

}  // namespace bnn
