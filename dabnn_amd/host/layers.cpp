#include "layers.h"

#include <sstream>
#include <stdexcept>

#include "../../include/dabnn_hip_tuning.h"
#include "net.h"

namespace bnn {

void bnn_fail(const std::string &msg) { throw std::runtime_error(msg); }

void dab_check(int rc) {
    if (rc != DAB_OK) throw std::runtime_error(dab_last_error());
}

// The kernels write n * oh * ow * c elements computed from the input and the window: the output blob a layer was
// handed must have exactly that geometry (a blob of another layer under the same name would be smaller).
static void check_window_output(const char *layer, const Mat &in, const Mat &out, int kh, int kw, int pad_h, int pad_w,
                                int stride_h, int stride_w, int dil_h, int dil_w, int channels) {
    BNN_ASSERT(stride_h > 0 && stride_w > 0 && pad_h >= 0 && pad_w >= 0 && kh > 0 && kw > 0, std::string(layer) + ": bad window");
    const long long oh = ((long long)in.h + 2ll * pad_h - ((long long)dil_h * (kh - 1) + 1)) / stride_h + 1;
    const long long ow = ((long long)in.w + 2ll * pad_w - ((long long)dil_w * (kw - 1) + 1)) / stride_w + 1;
    BNN_ASSERT(out.data_type == DataType::Float && out.n == in.n && out.h == oh && out.w == ow && out.c == channels,
               std::string(layer) + " output blob " + out.name + " is " + std::to_string(out.n) + "x" + std::to_string(out.h) + "x" +
                   std::to_string(out.w) + "x" + std::to_string(out.c) + ", the layer makes " + std::to_string(in.n) + "x" +
                   std::to_string(oh) + "x" + std::to_string(ow) + "x" + std::to_string(channels));
}

// ---------------------------------------------------------------- Layer
Layer::~Layer() {}

Layer::MatP Layer::mat(const std::string &name) const { return net_.lock()->blob(name); }

void *Layer::stream() const { return net_.lock()->stream(); }

std::string Layer::to_str() const { return type_ + " " + name_; }

// ---------------------------------------------------------------- BinConv
// dabnn/layers/BinConv.cpp:17-78: scratch blobs are registered in the net's
// blob map under the reference's names; the weights are transposed once for
// the bgemm method (:59-76).  No padded copy is kept: the direct kernel reads
// out-of-image taps as zero words itself.
BinConv::BinConv(NetCP net, css name, css input, css weight, css output, int pad_h_, int pad_w_, int stride_h_,
                 int stride_w_)
    : Layer(net, name, "Bin Conv"),
      input_mat(mat(input)),
      weight_mat(mat(weight)),
      output_mat(mat(output)),
      pad_h(pad_h_),
      pad_w(pad_w_),
      stride_h(stride_h_),
      stride_w(stride_w_) {
    auto n = net.lock();
    BNN_ASSERT(input_mat->data_type == DataType::Float, "BinConv input must be float");
    BNN_ASSERT(weight_mat->data_type == DataType::Bit, "BinConv weight must be Bit");
    BNN_ASSERT(input_mat->elem_c % 64 == 0, "BinConv needs a multiple of 64 input channels, got " +
                                                std::to_string(input_mat->elem_c));
    BNN_ASSERT(weight_mat->n > 0 && weight_mat->total() % weight_mat->n == 0, "weight size is not a multiple of the filter count");
    // the kernels take every extent from the input and the filter count: a weight tensor that is shorter than that
    // geometry says would be read past its end
    BNN_ASSERT(weight_mat->elem_c == input_mat->elem_c, "BinConv weight has " + std::to_string(weight_mat->elem_c) +
                                                            " input channels, the input blob " + std::to_string(input_mat->elem_c));
    {
        const size_t per = weight_mat->total() / weight_mat->n;
        const size_t bits = (size_t)kernel_h() * kernel_w() * input_mat->elem_c;
        BNN_ASSERT(per * 64 >= bits && per <= (size_t)dab_col_row_words(kernel_h(), kernel_w(), input_mat->elem_c),
                   "BinConv weight holds " + std::to_string(per) + " words per filter, its geometry needs " +
                       std::to_string((bits + 63) / 64));
        if (direct_conv_compatible())
            BNN_ASSERT(per == (size_t)9 * (input_mat->elem_c / 64), "BinConv weight holds " + std::to_string(per) +
                                                                        " words per filter, the direct 3x3 kernel walks " +
                                                                        std::to_string(9 * (input_mat->elem_c / 64)));
    }

    check_window_output("BinConv", *input_mat, *output_mat, kernel_h(), kernel_w(), pad_h, pad_w, stride_h, stride_w, 1, 1,
                        weight_mat->n);

    const std::string binarized_name = "binaized_for_" + output + "_cal";
    if (!n->has_blob(binarized_name))
        n->add_mat(binarized_name, std::make_shared<Mat>(input_mat->n, input_mat->h, input_mat->w, input_mat->elem_c,
                                                         DataType::Bit, binarized_name));
    binarized_mat = mat(binarized_name);
    BNN_ASSERT(binarized_mat->data_type == DataType::Bit &&
                   binarized_mat->total() >= (size_t)input_mat->n * input_mat->h * input_mat->w * (input_mat->elem_c / 64),
               "blob " + binarized_name + " is too small for the packed input");

    const std::string col_name = "col_for_" + output + "_cal";
    if (!n->has_blob(col_name)) {
        const size_t len = (size_t)output_mat->n * output_mat->h * output_mat->w *
                           dab_col_row_words(kernel_h(), kernel_w(), input_mat->elem_c);
        n->add_mat(col_name, std::make_shared<Mat>(len, DataType::Bit, col_name));
    }
    col_mat = mat(col_name);
    BNN_ASSERT(col_mat->data_type == DataType::Bit &&
                   col_mat->total() >= (size_t)output_mat->n * output_mat->h * output_mat->w *
                                           dab_col_row_words(kernel_h(), kernel_w(), input_mat->elem_c),
               "blob " + col_name + " is too small for the column matrix");

    const int m = weight_mat->n;
    const int k = (int)(weight_mat->total() / m);
    transposed_weight_mat = std::make_shared<Mat>((size_t)m * k, DataType::Bit, "trans_" + weight);
    dab_check(dab_weight_transpose(static_cast<const uint64_t *>(weight_mat->dev), m, k,
                                   static_cast<uint64_t *>(transposed_weight_mat->dev), n->stream()));
    n->add_mat("trans_" + weight, transposed_weight_mat);
}

bool BinConv::direct_conv_compatible() const {
    // dabnn/layers/BinConv.cpp:100-126
    const int c = input_mat->elem_c;
    return kernel_h() == 3 && kernel_w() == 3 && stride_h == stride_w && pad_h == pad_w &&
           (c == 64 || c == 128 || c == 256 || c == 512 || c == 1024) && weight_mat->n % 8 == 0;
}

BinConv::Method BinConv::method() const {
    if (net_.lock()->optimize && direct_conv_compatible()) return DIRECT_CONV;
    return BGEMM;
}

void BinConv::forward_impl() const {
    void *s = stream();
    const auto *x = static_cast<const float *>(input_mat->dev);
    auto *out = static_cast<float *>(output_mat->dev);
    const int n = input_mat->n, h = input_mat->h, w = input_mat->w, c = input_mat->elem_c;
    switch (method()) {
        case DIRECT_CONV: {
            // pack_mat + (pad +) bconv_3x3, dabnn/layers/BinConv.cpp:146-150
            auto *packed = static_cast<uint64_t *>(binarized_mat->dev);
            if (!input_prepacked) dab_check(dab_bitpack_nhwc(x, packed, (int64_t)n * h * w, c, s));
            if (fused_a && fused_sign_out) {
                dab_check(dab_bconv3x3_affine_add_sign(
                    packed, n, h, w, c, static_cast<const uint64_t *>(weight_mat->dev), weight_mat->n, stride_h, pad_h,
                    static_cast<const float *>(fused_a->dev), static_cast<const float *>(fused_b->dev),
                    fused_shortcut ? static_cast<const float *>(fused_shortcut->dev) : nullptr, out,
                    static_cast<uint64_t *>(fused_sign_out->dev), s));
            } else if (fused_a) {
                dab_check(dab_bconv3x3_affine_add(
                    packed, n, h, w, c, static_cast<const uint64_t *>(weight_mat->dev), weight_mat->n, stride_h, pad_h,
                    static_cast<const float *>(fused_a->dev), static_cast<const float *>(fused_b->dev),
                    fused_shortcut ? static_cast<const float *>(fused_shortcut->dev) : nullptr, out, s));
            } else {
                dab_check(dab_bconv3x3(packed, n, h, w, c, static_cast<const uint64_t *>(weight_mat->dev), weight_mat->n,
                                       stride_h, pad_h, out, s));
            }
            break;
        }
        case BGEMM: {
            // fill + fused_binarize_im2col + bgemm, dabnn/layers/BinConv.cpp:152-165; the fill and the accumulation
            // into it are one store (0.f + count == count)
            auto *col = static_cast<uint64_t *>(col_mat->dev);
            dab_check(dab_fused_binarize_im2col(x, n, h, w, c, kernel_h(), kernel_w(), pad_h, pad_w, stride_h, stride_w, 1,
                                                1, col, s));
            const int m = weight_mat->n;
            const int cols = n * output_mat->h * output_mat->w;
            const int k = (int)(weight_mat->total() / m);
            const int ldb = dab_col_row_words(kernel_h(), kernel_w(), c);  // rows are padded to 128 bits
            dab_check(dab_bgemm_overwrite(m, cols, k, static_cast<const uint64_t *>(transposed_weight_mat->dev), m, col, ldb,
                                          out, m, s));
            break;
        }
    }
}

std::string BinConv::to_str() const {
    std::stringstream ss;
    ss << type_ << ", input " << input_mat->h << "x" << input_mat->w << "x" << input_mat->elem_c << ", weight "
       << weight_mat->n << "x" << kernel_h() << "x" << kernel_w() << ", pad " << pad_h << "," << pad_w << ", stride "
       << stride_h << "," << stride_w << ", method " << (method() == DIRECT_CONV ? "DIRECT_CONV" : "BGEMM");
    if (input_prepacked) ss << ", packed input from its producer";
    if (fused_a) ss << (fused_shortcut ? " + Affine + Add" : " + Affine");
    if (fused_sign_out) ss << " + Sign";
    return ss.str();
}

// ---------------------------------------------------------------- FloatConv
FloatConv::FloatConv(NetCP net, css name, css input, css weight, css bias, css output, int pad_h_, int pad_w_,
                     int stride_h_, int stride_w_, int dilation_)
    : Layer(net, name, "Float Conv"),
      input_mat(mat(input)),
      weight_mat(mat(weight)),
      bias_mat(mat(bias)),
      output_mat(mat(output)),
      pad_h(pad_h_),
      pad_w(pad_w_),
      stride_h(stride_h_),
      stride_w(stride_w_),
      dilation(dilation_) {
    check_operands();
}

FloatConv::FloatConv(NetCP net, css name, css input, css weight, css output, int pad_h_, int pad_w_, int stride_h_,
                     int stride_w_, int dilation_)
    : Layer(net, name, "Float Conv"),
      input_mat(mat(input)),
      weight_mat(mat(weight)),
      output_mat(mat(output)),
      pad_h(pad_h_),
      pad_w(pad_w_),
      stride_h(stride_h_),
      stride_w(stride_w_),
      dilation(dilation_) {
    check_operands();
}

// The kernel sizes its weight descriptor as cout * kh * kw * input channels: the tensors must say the same.
void FloatConv::check_operands() const {
    BNN_ASSERT(input_mat->data_type == DataType::Float && weight_mat->data_type == DataType::Float, "FloatConv operands must be float");
    BNN_ASSERT(weight_mat->c == input_mat->c, "FloatConv weight has " + std::to_string(weight_mat->c) +
                                                  " input channels, the input blob " + std::to_string(input_mat->c));
    BNN_ASSERT(weight_mat->total() == (size_t)weight_mat->n * weight_mat->h * weight_mat->w * input_mat->c,
               "FloatConv weight does not match its shape");
    BNN_ASSERT(output_mat->c == weight_mat->n, "FloatConv output does not have one channel per filter");
    if (bias_mat) BNN_ASSERT((int)bias_mat->total() == weight_mat->n, "FloatConv bias does not match the filter count");
    BNN_ASSERT(stride_h > 0 && stride_w > 0 && dilation > 0 && pad_h >= 0 && pad_w >= 0, "FloatConv: bad stride, dilation or pad");
    check_window_output("FloatConv", *input_mat, *output_mat, weight_mat->h, weight_mat->w, pad_h, pad_w, stride_h, stride_w,
                        dilation, dilation, weight_mat->n);
}

void FloatConv::forward_impl() const {
    if (fused_pool_input) {
        dab_check((fused_pool_global ? dab_global_ave_pool_fconv1x1 : dab_ave_pool2_fconv1x1)(
            static_cast<const float *>(fused_pool_input->dev), fused_pool_input->n, fused_pool_input->h, fused_pool_input->w,
            fused_pool_input->c, static_cast<const float *>(weight_mat->dev),
            bias_mat ? static_cast<const float *>(bias_mat->dev) : nullptr,
            fused_a ? static_cast<const float *>(fused_a->dev) : nullptr,
            fused_b ? static_cast<const float *>(fused_b->dev) : nullptr, fused_relu ? 1 : 0, output_mat->c,
            static_cast<float *>(input_mat->dev), static_cast<float *>(output_mat->dev), stream()));
        return;
    }
    if (fused_maxpool_out) {
        dab_check(dab_fconv_maxpool(
            static_cast<const float *>(input_mat->dev), input_mat->n, input_mat->h, input_mat->w, input_mat->c,
            static_cast<const float *>(weight_mat->dev), bias_mat ? static_cast<const float *>(bias_mat->dev) : nullptr,
            fused_a ? static_cast<const float *>(fused_a->dev) : nullptr,
            fused_b ? static_cast<const float *>(fused_b->dev) : nullptr, fused_relu ? 1 : 0, weight_mat->h, weight_mat->w,
            pad_h, pad_w, stride_h, stride_w, dilation, dilation, weight_mat->n, static_cast<float *>(fused_maxpool_out->dev),
            fused_maxpool_sign ? static_cast<uint64_t *>(fused_maxpool_sign->dev) : nullptr,
            static_cast<float *>(fused_maxpool_carry->dev), stream()));
        return;
    }
    dab_check(dab_fconv_affine_relu(
        static_cast<const float *>(input_mat->dev), input_mat->n, input_mat->h, input_mat->w, input_mat->c,
        static_cast<const float *>(weight_mat->dev), bias_mat ? static_cast<const float *>(bias_mat->dev) : nullptr,
        fused_a ? static_cast<const float *>(fused_a->dev) : nullptr,
        fused_b ? static_cast<const float *>(fused_b->dev) : nullptr, fused_relu ? 1 : 0, weight_mat->h, weight_mat->w,
        pad_h, pad_w, stride_h, stride_w, dilation, dilation, output_mat->c, static_cast<float *>(output_mat->dev),
        stream()));
}

std::string FloatConv::to_str() const {
    std::stringstream ss;
    ss << type_ << ", input " << input_mat->h << "x" << input_mat->w << "x" << input_mat->c << ", weight " << weight_mat->n
       << "x" << weight_mat->h << "x" << weight_mat->w;
    if (fused_a) ss << " + Affine";
    if (fused_relu) ss << " + Relu";
    if (fused_pool_input)
        ss << ", AvePool " << (fused_pool_global ? "over all" : "2x2") << " of " << fused_pool_input->h << "x" << fused_pool_input->w << " inside";
    if (fused_maxpool_out) ss << " + MaxPool 3x3 stride 2" << (fused_maxpool_sign ? " + Sign" : "");
    return ss.str();
}

// ---------------------------------------------------------------- Affine / Add / Relu (in place)
Affine::Affine(NetCP net, css name, css data, css a, css b)
    : Layer(net, name, "Affine"), data_mat(mat(data)), a_mat(mat(a)), b_mat(mat(b)) {
    BNN_ASSERT((int)a_mat->total() == data_mat->c && (int)b_mat->total() == data_mat->c,
               "Affine coefficients do not match the channel count");
}

void Affine::forward_impl() const {
    dab_check(dab_affine_inplace(static_cast<float *>(data_mat->dev), (int64_t)data_mat->n * data_mat->h * data_mat->w,
                                 data_mat->c, static_cast<const float *>(a_mat->dev),
                                 static_cast<const float *>(b_mat->dev), stream()));
}

Add::Add(NetCP net, css name, css input1, css input2)
    : Layer(net, name, "Add"), input1_mat(mat(input1)), input2_mat(mat(input2)) {
    BNN_ASSERT(input1_mat->total() == input2_mat->total(), "Add operands differ in size");
}

void Add::forward_impl() const {
    dab_check(dab_add_inplace(static_cast<float *>(input1_mat->dev), static_cast<const float *>(input2_mat->dev),
                              (int64_t)input1_mat->total(), stream()));
}

Relu::Relu(NetCP net, css name, css data) : Layer(net, name, "Relu"), data_mat(mat(data)) {}

void Relu::forward_impl() const {
    dab_check(dab_relu_inplace(static_cast<float *>(data_mat->dev), (int64_t)data_mat->total(), stream()));
}

// dabnn/layers/PRelu.cpp:6-30; the size check is the reference's, made once at construction
PRelu::PRelu(NetCP net, css name, css data, css slope)
    : Layer(net, name, "PRelu"), data_mat(mat(data)), slope_mat(mat(slope)) {
    BNN_ASSERT(slope_mat->total() == 1 || (int)slope_mat->total() == data_mat->c,
               "slope must have size 1 or input.channels");
}

void PRelu::forward_impl() const {
    dab_check(dab_prelu_inplace(static_cast<float *>(data_mat->dev), (int64_t)data_mat->n * data_mat->h * data_mat->w,
                                data_mat->c, static_cast<const float *>(slope_mat->dev), (int)slope_mat->total(), stream()));
}

// dabnn/layers/Concat.cpp:7-21 (two inputs, channel axis)
Concat::Concat(NetCP net, css name, css input1, css input2, css output)
    : Layer(net, name, "Concat"), input1_mat(mat(input1)), input2_mat(mat(input2)), output_mat(mat(output)) {
    BNN_ASSERT(input1_mat->n == input2_mat->n && input1_mat->h == input2_mat->h && input1_mat->w == input2_mat->w,
               "Wrong input for concat");
    BNN_ASSERT(output_mat->c == input1_mat->c + input2_mat->c, "Concat output does not hold both inputs");
}

void Concat::forward_impl() const {
    dab_check(dab_concat_channels(static_cast<const float *>(input1_mat->dev), input1_mat->c,
                                  static_cast<const float *>(input2_mat->dev), input2_mat->c,
                                  (int64_t)input1_mat->n * input1_mat->h * input1_mat->w,
                                  static_cast<float *>(output_mat->dev), stream()));
}

// ---------------------------------------------------------------- Split / Shuffle (Bit blobs)
Split::Split(NetCP net, css name, css input, css output1, css output2)
    : Layer(net, name, "Split"), input_mat(mat(input)), output_mat1(mat(output1)), output_mat2(mat(output2)) {
    BNN_ASSERT(input_mat->data_type == DataType::Bit, "Split only supports bit mat");  // dabnn/layers/Split.h:19-23
    BNN_ASSERT(input_mat->elem_c % 128 == 0 && input_mat->elem_c <= 512, "Split: " + std::to_string(input_mat->elem_c) + " channels");
    BNN_ASSERT(output_mat1->data_type == DataType::Bit && output_mat2->data_type == DataType::Bit &&
                   output_mat1->total() * 2 == input_mat->total() && output_mat2->total() * 2 == input_mat->total(),
               "Split outputs must each hold half of the input's words");
}

void Split::forward_impl() const {
    dab_check(dab_split_bit(static_cast<const uint64_t *>(input_mat->dev), (int64_t)(input_mat->total() / input_mat->c), input_mat->c,
                            static_cast<uint64_t *>(output_mat1->dev), static_cast<uint64_t *>(output_mat2->dev), stream()));
}

Shuffle::Shuffle(NetCP net, css name, css data) : Layer(net, name, "Shuffle"), data_mat(mat(data)) {
    BNN_ASSERT(data_mat->data_type == DataType::Bit, "Shuffle only supports bit mat");  // dabnn/layers/Shuffle.h:16-20
    BNN_ASSERT(data_mat->elem_c % 128 == 0 && data_mat->elem_c <= 512, "Shuffle: " + std::to_string(data_mat->elem_c) + " channels");
}

void Shuffle::forward_impl() const {
    dab_check(dab_shuffle_bit_inplace(static_cast<uint64_t *>(data_mat->dev), (int64_t)(data_mat->total() / data_mat->c),
                                      data_mat->elem_c, stream()));
}

// ---------------------------------------------------------------- pooling
AvePool::AvePool(NetCP net, css name, css input, css output, int kernel_h_, int kernel_w_, int pad_h_, int pad_w_,
                 int stride_h_, int stride_w_)
    : Layer(net, name, "AvePool"),
      input_mat(mat(input)),
      output_mat(mat(output)),
      kernel_h(kernel_h_),
      kernel_w(kernel_w_),
      pad_h(pad_h_),
      pad_w(pad_w_),
      stride_h(stride_h_),
      stride_w(stride_w_) {
    BNN_ASSERT(input_mat->data_type == DataType::Float, "pooling input must be float");
    check_window_output("AvePool", *input_mat, *output_mat, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w, 1, 1, input_mat->c);
}

void AvePool::forward_impl() const {
    dab_check(dab_ave_pool(static_cast<const float *>(input_mat->dev), input_mat->n, input_mat->h, input_mat->w,
                           input_mat->c, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w,
                           static_cast<float *>(output_mat->dev), stream()));
}

MaxPool::MaxPool(NetCP net, css name, css input, css output, int kernel_h_, int kernel_w_, int pad_h_, int pad_w_,
                 int stride_h_, int stride_w_)
    : Layer(net, name, "MaxPool"),
      input_mat(mat(input)),
      output_mat(mat(output)),
      kernel_h(kernel_h_),
      kernel_w(kernel_w_),
      pad_h(pad_h_),
      pad_w(pad_w_),
      stride_h(stride_h_),
      stride_w(stride_w_) {
    BNN_ASSERT(input_mat->data_type == DataType::Float, "pooling input must be float");
    check_window_output("MaxPool", *input_mat, *output_mat, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w, 1, 1, input_mat->c);
}

void MaxPool::forward_impl() const {
    if (fused_sign_out) {
        dab_check(dab_max_pool_sign(static_cast<const float *>(input_mat->dev), input_mat->n, input_mat->h, input_mat->w,
                                    input_mat->c, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w,
                                    static_cast<float *>(output_mat->dev), static_cast<uint64_t *>(fused_sign_out->dev),
                                    stream()));
        return;
    }
    dab_check(dab_max_pool(static_cast<const float *>(input_mat->dev), input_mat->n, input_mat->h, input_mat->w,
                           input_mat->c, kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w,
                           static_cast<float *>(output_mat->dev), stream()));
}

}  // namespace bnn
