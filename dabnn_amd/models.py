"""Random-init Bi-Real-Net-18 style models in dabnn's layer vocabulary.

The pretrained models of the reference are not redistributable here, so
benchmarks and tests use synthetic networks with the same graph: what the
reference's converter would emit for Bi-Real-18 (tools/onnx2bnn/OnnxConverter.cpp
and docs/onnx2bnn.md): weights transposed to [Cout, KH, KW, Cin], binary
weights sign-packed along (KH, KW, Cin) with every filter zero-bit padded to a
multiple of 128 bits unless Cin == 64 (OnnxConverter.cpp:121-156), batch norm
folded into a per-channel affine with a' = -2a, b' = b + K*a after a binary
convolution (:583-639), the FC layer expressed as a 1x1 float convolution.

Graph (NHWC):
  input 224x224x3
  stem: FpConv2D 7x7 s2 p3 (3->64) + Affine           [variant: three 3x3 convs 32/32/64, first one stride 2,
                                                        each + Affine + Relu]
  MaxPool 3x3 s2 p1 -> 56x56x64
  16 blocks of  BinConv2D 3x3 -> Affine -> Add(shortcut)
      stages of 4 blocks at 64/128/256/512 channels; the first block of stages
      2-4 has stride 2 and its shortcut is AvePool 2x2 s2 -> FpConv2D 1x1 -> Affine
  AvePool 7x7 -> FpConv2D 1x1 (512->1000, with bias)
"""
import numpy as np


def pack_bits(x):
    """float [..., n*64] -> uint64 [..., n]; bit j of word i = (x[64 i + j] > 0)."""
    bits = np.asarray(x, dtype=np.float32) > 0
    return np.packbits(bits, axis=-1, bitorder="little").view("<u8")


def pack_weight(wf):
    """fp32 [Cout, KH, KW, Cin] -> uint64 [Cout, words]: the converter's bitpack rule."""
    cout, kh, kw, c = wf.shape
    flat = wf.reshape(cout, kh * kw * c)
    if c != 64:
        pad = (-flat.shape[1]) % 128
        flat = np.pad(flat, ((0, 0), (0, pad)), constant_values=-1.0)  # padding bits are 0
    return np.ascontiguousarray(pack_bits(flat))


def fold_bn(scale, bias, mean, var, eps=1e-5, k_bits=0):
    """Batch norm -> (a, b) of an Affine layer; k_bits > 0 when it follows a binary convolution."""
    t = np.sqrt(var.astype(np.float32) + np.float32(eps)).astype(np.float32)
    a = (scale / t).astype(np.float32)
    b = (bias - scale * mean / t).astype(np.float32)
    if k_bits:
        b = (b + np.float32(k_bits) * a).astype(np.float32)
        a = (a * np.float32(-2)).astype(np.float32)
    return a, b


def bireal18(seed=0, stem=False, num_classes=1000):
    """Returns (layers, initializers, inputs) for dab_format.write_model."""
    r = np.random.default_rng(seed)
    layers, inits = [], []

    def tensor(name, data, shape=None, align=False):
        inits.append({"name": name, "shape": list(data.shape if shape is None else shape), "data": data,
                      "align_hwc_to_128": align})
        return name

    def bn(prefix, c, k_bits=0, gain=1.0):
        scale = (gain * (1.0 + 0.1 * r.standard_normal(c))).astype(np.float32)
        bias = (0.1 * r.standard_normal(c)).astype(np.float32)
        mean = (0.1 * r.standard_normal(c)).astype(np.float32)
        var = r.uniform(0.8, 1.2, c).astype(np.float32)
        if k_bits:  # conv(sign x, sign w) has variance ~ k_bits: normalise to O(1)
            mean = (mean * np.sqrt(k_bits)).astype(np.float32)
            var = (var * k_bits).astype(np.float32)
        a, b = fold_bn(scale, bias, mean, var, 1e-5, k_bits)
        return tensor(prefix + "_a", a), tensor(prefix + "_b", b)

    def fconv(name, src, dst, cin, cout, k, stride, pad, bias=False):
        w = (r.standard_normal((cout, k, k, cin)) / np.sqrt(k * k * cin)).astype(np.float32)
        layer = {"type": "FpConv2D", "name": name, "input": src, "weight": tensor(name + "_w", w), "output": dst,
                 "pads": [pad] * 4, "strides": [stride, stride], "dilations": [1, 1]}
        if bias:
            layer["bias"] = tensor(name + "_bias", (0.1 * r.standard_normal(cout)).astype(np.float32))
        layers.append(layer)

    def affine(name, blob, a, b):
        layers.append({"type": "Affine", "name": name, "input": blob, "a": a, "b": b, "output": blob + "_bn"})
        return blob + "_bn"

    if stem:
        cur, cin = "data", 3
        for i, (cout, stride) in enumerate([(32, 2), (32, 1), (64, 1)]):
            fconv("stem%d" % i, cur, "stem%d_out" % i, cin, cout, 3, stride, 1)
            a, b = bn("stem%d_bn" % i, cout)
            cur = affine("stem%d_affine" % i, "stem%d_out" % i, a, b)
            layers.append({"type": "Relu", "name": "stem%d_relu" % i, "input": cur, "output": cur + "_relu"})
            cur, cin = cur + "_relu", cout
    else:
        fconv("conv1", "data", "conv1_out", 3, 64, 7, 2, 3)
        a, b = bn("bn1", 64)
        cur = affine("bn1_affine", "conv1_out", a, b)
    layers.append({"type": "MaxPool", "name": "pool1", "input": cur, "output": "pool1_out", "kernel_shape": [3, 3],
                   "pads": [1, 1, 1, 1], "strides": [2, 2]})
    cur, cin = "pool1_out", 64

    for stage, cout in enumerate([64, 128, 256, 512]):
        for block in range(4):
            p = "s%db%d" % (stage + 1, block)
            stride = 2 if (stage > 0 and block == 0) else 1
            wf = r.standard_normal((cout, 3, 3, cin)).astype(np.float32)
            wname = tensor(p + "_w", pack_weight(wf).ravel(), shape=[cout, 3, 3, cin], align=(cin != 64))
            layers.append({"type": "BinConv2D", "name": p + "_bconv", "input": cur, "weight": wname,
                           "output": p + "_cnt", "pads": [1, 1, 1, 1], "strides": [stride, stride], "dilations": [1, 1]})
            a, b = bn(p + "_bn", cout, k_bits=9 * cin, gain=0.5)
            main = affine(p + "_affine", p + "_cnt", a, b)
            shortcut = cur
            if stride == 2:
                layers.append({"type": "AvePool", "name": p + "_sc_pool", "input": cur, "output": p + "_sc_pool_out",
                               "kernel_shape": [2, 2], "pads": [0, 0, 0, 0], "strides": [2, 2]})
                fconv(p + "_sc_conv", p + "_sc_pool_out", p + "_sc_conv_out", cin, cout, 1, 1, 0)
                sa, sb = bn(p + "_sc_bn", cout)
                shortcut = affine(p + "_sc_affine", p + "_sc_conv_out", sa, sb)
            layers.append({"type": "Add", "name": p + "_add", "input1": main, "input2": shortcut, "output": p + "_out"})
            cur, cin = p + "_out", cout

    layers.append({"type": "AvePool", "name": "pool5", "input": cur, "output": "pool5_out", "kernel_shape": [7, 7],
                   "pads": [0, 0, 0, 0], "strides": [1, 1]})
    fconv("fc", "pool5_out", "logits", 512, num_classes, 1, 1, 0, bias=True)
    return layers, inits, [("data", [1, 224, 224, 3])]


def small_bnn(seed=0, hw=16, width=64):
    """A four-block miniature of the same graph for quick tests (input hw x hw x 3).

    With width 64 the blocks see 64, 64, 128 and 192 input channels, so both the direct 3x3 kernel and the
    im2col + bgemm method (192 channels) run."""
    r = np.random.default_rng(seed)
    layers, inits = [], []

    def tensor(name, data, shape=None, align=False):
        inits.append({"name": name, "shape": list(data.shape if shape is None else shape), "data": data,
                      "align_hwc_to_128": align})
        return name

    w = (r.standard_normal((width, 3, 3, 3)) / np.sqrt(27)).astype(np.float32)
    layers.append({"type": "FpConv2D", "name": "conv1", "input": "data", "weight": tensor("conv1_w", w),
                   "output": "conv1_out", "pads": [1] * 4, "strides": [1, 1], "dilations": [1, 1]})
    cur, cin = "conv1_out", width
    for i, (cout, stride) in enumerate([(width, 1), (2 * width, 2), (3 * width, 1), (3 * width, 1)]):
        p = "b%d" % i
        wf = r.standard_normal((cout, 3, 3, cin)).astype(np.float32)
        wname = tensor(p + "_w", pack_weight(wf).ravel(), shape=[cout, 3, 3, cin], align=(cin != 64))
        layers.append({"type": "BinConv2D", "name": p + "_bconv", "input": cur, "weight": wname, "output": p + "_cnt",
                       "pads": [1] * 4, "strides": [stride, stride], "dilations": [1, 1]})
        a, b = fold_bn(np.full(cout, 0.5, np.float32), (0.1 * r.standard_normal(cout)).astype(np.float32),
                       np.zeros(cout, np.float32), np.full(cout, 9.0 * cin, np.float32), 1e-5, 9 * cin)
        layers.append({"type": "Affine", "name": p + "_affine", "input": p + "_cnt", "a": tensor(p + "_a", a),
                       "b": tensor(p + "_b", b), "output": p + "_bn"})
        if stride == 1 and cout == cin:
            layers.append({"type": "Add", "name": p + "_add", "input1": p + "_bn", "input2": cur, "output": p + "_out"})
            cur = p + "_out"
        else:
            cur = p + "_bn"
        cin = cout
    layers.append({"type": "AvePool", "name": "gap", "input": cur, "output": "gap_out",
                   "kernel_shape": [hw // 2, hw // 2], "pads": [0] * 4, "strides": [1, 1]})
    wfc = (r.standard_normal((10, 1, 1, cin)) / np.sqrt(cin)).astype(np.float32)
    layers.append({"type": "FpConv2D", "name": "fc", "input": "gap_out", "weight": tensor("fc_w", wfc),
                   "bias": tensor("fc_bias", (0.1 * r.standard_normal(10)).astype(np.float32)), "output": "logits",
                   "pads": [0] * 4, "strides": [1, 1], "dilations": [1, 1]})
    return layers, inits, [("data", [1, hw, hw, 3])]


def dense_bnn(seed=0, hw=16, growth=64):
    """A BiDenseNet-style miniature (input hw x hw x 3) in the layer vocabulary the converter emits for such nets
    (tools/onnx2bnn/OnnxConverter.cpp:373-400 PRelu, :490-513 Concat):

      FpConv2D 3x3 (3 -> growth) + Affine + PRelu (one slope per channel)
      dense block: 3 x [BinConv2D 3x3 (cin -> growth) + Affine, Concat(features, new)]   cin = g, 2g, 3g
      transition:  MaxPool 2x2 s2, FpConv2D 1x1 (4g -> 2g) + Affine + PRelu (one slope)
      dense block: 2 x [BinConv2D 3x3 + Affine, Concat]                                   cin = 2g, 3g
      AvePool (global) + FpConv2D 1x1 with bias (4g -> 10)

    With growth 64 the binary convolutions see 64, 128, 192, 128 and 192 input channels: the direct 3x3 kernel and the
    im2col + bgemm method with a filter padded to a multiple of 128 bits both run."""
    r = np.random.default_rng(seed)
    layers, inits = [], []

    def tensor(name, data, shape=None, align=False):
        inits.append({"name": name, "shape": list(data.shape if shape is None else shape), "data": data,
                      "align_hwc_to_128": align})
        return name

    def fconv(name, src, dst, cin, cout, k, pad, bias=False):
        w = (r.standard_normal((cout, k, k, cin)) / np.sqrt(k * k * cin)).astype(np.float32)
        layer = {"type": "FpConv2D", "name": name, "input": src, "weight": tensor(name + "_w", w), "output": dst,
                 "pads": [pad] * 4, "strides": [1, 1], "dilations": [1, 1]}
        if bias:
            layer["bias"] = tensor(name + "_bias", (0.1 * r.standard_normal(cout)).astype(np.float32))
        layers.append(layer)

    def affine_prelu(p, blob, c, per_channel):
        a = (1.0 + 0.1 * r.standard_normal(c)).astype(np.float32)
        b = (0.1 * r.standard_normal(c)).astype(np.float32)
        layers.append({"type": "Affine", "name": p + "_affine", "input": blob, "a": tensor(p + "_a", a),
                       "b": tensor(p + "_b", b), "output": blob + "_bn"})
        slope = r.uniform(0.1, 0.4, c if per_channel else 1).astype(np.float32)
        layers.append({"type": "PRelu", "name": p + "_prelu", "input": blob + "_bn", "slope": tensor(p + "_slope", slope),
                       "output": blob + "_act"})
        return blob + "_act"

    def dense_layer(p, cur, cin):
        wf = r.standard_normal((growth, 3, 3, cin)).astype(np.float32)
        wname = tensor(p + "_w", pack_weight(wf).ravel(), shape=[growth, 3, 3, cin], align=(cin != 64))
        layers.append({"type": "BinConv2D", "name": p + "_bconv", "input": cur, "weight": wname, "output": p + "_cnt",
                       "pads": [1] * 4, "strides": [1, 1], "dilations": [1, 1]})
        a, b = fold_bn(np.full(growth, 0.5, np.float32), (0.1 * r.standard_normal(growth)).astype(np.float32),
                       np.zeros(growth, np.float32), np.full(growth, 9.0 * cin, np.float32), 1e-5, 9 * cin)
        layers.append({"type": "Affine", "name": p + "_affine", "input": p + "_cnt", "a": tensor(p + "_a", a),
                       "b": tensor(p + "_b", b), "output": p + "_bn"})
        layers.append({"type": "Concat", "name": p + "_concat", "inputs": [cur, p + "_bn"], "axis": 3,
                       "output": p + "_cat"})
        return p + "_cat", cin + growth

    fconv("conv1", "data", "conv1_out", 3, growth, 3, 1)
    cur, cin = affine_prelu("stem", "conv1_out", growth, True), growth
    for i in range(3):
        cur, cin = dense_layer("d1l%d" % i, cur, cin)
    layers.append({"type": "MaxPool", "name": "t1_pool", "input": cur, "output": "t1_pool_out", "kernel_shape": [2, 2],
                   "pads": [0] * 4, "strides": [2, 2]})
    fconv("t1_conv", "t1_pool_out", "t1_conv_out", cin, cin // 2, 1, 0)
    cur, cin = affine_prelu("t1", "t1_conv_out", cin // 2, False), cin // 2
    for i in range(2):
        cur, cin = dense_layer("d2l%d" % i, cur, cin)
    layers.append({"type": "AvePool", "name": "gap", "input": cur, "output": "gap_out",
                   "kernel_shape": [hw // 2, hw // 2], "pads": [0] * 4, "strides": [1, 1]})
    fconv("fc", "gap_out", "logits", cin, 10, 1, 0, bias=True)
    return layers, inits, [("data", [1, hw, hw, 3])]
