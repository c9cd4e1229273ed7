// The layers Net::prepare of the reference builds (dabnn/layers/{BinConv,FloatConv,
// Affine,Add,AvePool,MaxPool,Relu,PRelu,Concat,Split,Shuffle}.{h,cpp}); constructor
// signatures follow the reference.
#pragma once

#include "layer.h"

namespace bnn {

using css = const std::string &;

class BNN_API BinConv : public Layer {
   public:
    MatP input_mat;
    MatP binarized_mat;  // packed input of the direct method
    MatP col_mat;        // column matrix of the bgemm method
    MatP weight_mat;
    MatP transposed_weight_mat;
    MatP output_mat;
    const int pad_h, pad_w, stride_h, stride_w;

    enum Method { DIRECT_CONV = 0, BGEMM = 1 };

    // Set by Net::prepare when the layers that follow are Affine (and Add) on this layer's output and the direct
    // kernel applies: the three run as one pass with identical results.
    MatP fused_a, fused_b, fused_shortcut;
    // Also set by Net::prepare: the fused pass of this layer writes the sign-packed copy of its result that the next
    // direct BinConv on that blob needs (fused_sign_out = that layer's binarized_mat), and a layer whose packed input
    // is made that way skips its own pack_mat (input_prepacked).
    MatP fused_sign_out;
    bool input_prepacked = false;

    BinConv(NetCP net, css name, css input, css weight, css output, int pad_h, int pad_w, int stride_h, int stride_w);
    void forward_impl() const override;
    std::string to_str() const override;
    Method method() const;

   private:
    int kernel_h() const { return weight_mat->h; }
    int kernel_w() const { return weight_mat->w; }
    bool direct_conv_compatible() const;
};

class BNN_API FloatConv : public Layer {
   public:
    MatP input_mat, weight_mat, bias_mat, output_mat;
    // Affine (and Relu) layers that follow on the output blob, applied in the convolution's epilogue when set
    MatP fused_a, fused_b;
    bool fused_relu = false;
    // Set by Net::prepare for a 1x1 convolution that reads the output of an AvePool 2x2 stride 2: the pool's input.
    // The layer then pools it itself and convolves the result; the pooled blob (input_mat) is written as a side product
    // when it has device memory, and is a shape without memory when the net dropped the blob.
    MatP fused_pool_input;
    // The same for a global AvePool (one window over the whole image) at small batch: fused_pool_input is its input.
    bool fused_pool_global = false;
    // Set by Net::prepare when a MaxPool 3x3 stride 2 pad 1 is the only reader of the output: the pool's output blob,
    // the packed copy of it a direct BinConv wants (or null) and the workspace of the one-pass kernel.  output_mat is
    // null then: the convolution's result is never written.
    MatP fused_maxpool_out, fused_maxpool_sign, fused_maxpool_carry;
    const int pad_h, pad_w, stride_h, stride_w, dilation;
    FloatConv(NetCP net, css name, css input, css weight, css bias, css output, int pad_h, int pad_w, int stride_h,
              int stride_w, int dilation);
    FloatConv(NetCP net, css name, css input, css weight, css output, int pad_h, int pad_w, int stride_h, int stride_w,
              int dilation);
    void forward_impl() const override;
    std::string to_str() const override;

   private:
    void check_operands() const;
};

class BNN_API Affine : public Layer {
   public:
    MatP data_mat, a_mat, b_mat;
    Affine(NetCP net, css name, css data, css a, css b);
    void forward_impl() const override;
};

class BNN_API Add : public Layer {
   public:
    MatP input1_mat, input2_mat;
    Add(NetCP net, css name, css input1, css input2);
    void forward_impl() const override;
};

class BNN_API Relu : public Layer {
   public:
    MatP data_mat;
    Relu(NetCP net, css name, css data);
    void forward_impl() const override;
};

class BNN_API PRelu : public Layer {
   public:
    MatP data_mat, slope_mat;
    PRelu(NetCP net, css name, css data, css slope);
    void forward_impl() const override;
};

class BNN_API Concat : public Layer {
   public:
    MatP input1_mat, input2_mat, output_mat;
    Concat(NetCP net, css name, css input1, css input2, css output);
    void forward_impl() const override;
};

// dabnn/layers/Split.{h,cpp}: a Bit blob's words per pixel cut in two halves (first half -> output 1).
class BNN_API Split : public Layer {
   public:
    MatP input_mat, output_mat1, output_mat2;
    Split(NetCP net, css name, css input, css output1, css output2);
    void forward_impl() const override;
};

// dabnn/layers/Shuffle.{h,cpp}: the channel shuffle of a two-group network on packed words, in place.
class BNN_API Shuffle : public Layer {
   public:
    MatP data_mat;
    Shuffle(NetCP net, css name, css data);
    void forward_impl() const override;
};

class BNN_API AvePool : public Layer {
   public:
    MatP input_mat, output_mat;
    const int kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w;
    AvePool(NetCP net, css name, css input, css output, int kernel_h, int kernel_w, int pad_h, int pad_w, int stride_h,
            int stride_w);
    void forward_impl() const override;
};

class BNN_API MaxPool : public Layer {
   public:
    MatP input_mat, output_mat;
    // Set by Net::prepare when a direct BinConv reads the pooled blob: its packed input, written in the same pass.
    MatP fused_sign_out;
    const int kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w;
    MaxPool(NetCP net, css name, css input, css output, int kernel_h, int kernel_w, int pad_h, int pad_w, int stride_h,
            int stride_w);
    void forward_impl() const override;
};

}  // namespace bnn
