"""The .dab reader of the C++ Net on the host (no GPU): every FlatBuffers offset is checked against the buffer's
length, and the model's tensors are checked against its layers' geometry, before anything is built.

Reference behaviour kept: std::invalid_argument for unreadable input (dabnn/net.cpp:32-44), std::runtime_error from
BNN_ASSERT (common/helper.h:69-77) for models the reference would refuse while preparing (dabnn/net.cpp:56-270)."""
import struct

import numpy as np
import pytest

from dabnn_amd import dab_format as df
from dabnn_amd import models


@pytest.fixture(scope="module")
def net():
    from dabnn_amd import net
    return net


def small():
    layers, inits, inputs = models.small_bnn(0, hw=16, width=64)
    return layers, inits, inputs


def test_good_models_pass(net):
    net.check_model(df.write_model(*small()))
    for stem in (False, True):
        net.check_model(df.write_model(*models.bireal18(1, stem=stem)))
    net.check_model(df.write_model(*models.dense_bnn(2)))


def test_truncated_buffers_are_invalid_not_crashes(net):
    """Cut the file at every 64-byte boundary (and a few odd lengths): the root table sits at the front and points at
    strings and vectors all the way to the end, so every prefix that loses more than the final padding bytes (the
    last string here ends four bytes before the end of the file) must be refused as invalid."""
    buf = df.write_model(*small())
    assert buf[-4:] == b"\x00" * 4
    cuts = list(range(8, len(buf), 64)) + [9, 13, len(buf) - 5, len(buf) - 7, len(buf) - 64]
    for n in cuts:
        with pytest.raises(ValueError, match="malformed model buffer"):
            net.check_model(buf[:n])
    with pytest.raises(ValueError, match="too small"):
        net.check_model(buf[:4])


def test_corrupt_offsets_are_invalid(net):
    buf = bytearray(df.write_model(*small()))
    root = struct.unpack_from("<I", buf, 0)[0]
    # root offset beyond the buffer
    bad = bytearray(buf)
    struct.pack_into("<I", bad, 0, len(buf) + 1000)
    with pytest.raises(ValueError, match="malformed"):
        net.check_model(bad)
    # the root table's vtable offset pointing far outside (before the buffer / after it)
    for off in (len(buf) * 4, -(len(buf) * 4)):
        bad = bytearray(buf)
        struct.pack_into("<i", bad, root, off)
        with pytest.raises(ValueError, match="malformed"):
            net.check_model(bad)
    # a vtable that claims to be longer than the buffer
    vt = root - struct.unpack_from("<i", buf, root)[0]
    bad = bytearray(buf)
    struct.pack_into("<H", bad, vt, 0xFFF0)
    with pytest.raises(ValueError, match="malformed"):
        net.check_model(bad)
    # the layers vector's length field larger than the buffer
    f_layers = struct.unpack_from("<H", buf, vt + 4)[0]
    vec = root + f_layers + struct.unpack_from("<I", buf, root + f_layers)[0]
    bad = bytearray(buf)
    struct.pack_into("<I", bad, vec, 0x7FFFFFFF)
    with pytest.raises(ValueError, match="malformed"):
        net.check_model(bad)
    # a random flip of every 97th byte must never crash: any outcome but a fault is fine
    rng = np.random.default_rng(3)
    for trial in range(40):
        bad = bytearray(buf)
        for pos in rng.integers(0, len(buf), size=6):
            bad[pos] ^= int(rng.integers(1, 256))
        try:
            net.check_model(bad)
        except (ValueError, RuntimeError, KeyError):
            pass


def _binconv_model(c=128, cout=16, k=3, words=None, wc=None, stride=(1, 1), pads=(1, 1, 1, 1)):
    wc = c if wc is None else wc
    r = np.random.default_rng(5)
    wp = models.pack_weight(r.standard_normal((cout, k, k, wc)).astype(np.float32))
    if words is not None:
        wp = wp[:, :words] if words <= wp.shape[1] else np.concatenate([wp, np.zeros((cout, words - wp.shape[1]), np.uint64)], 1)
    inits = [{"name": "w", "shape": [cout, k, k, wc], "data": np.ascontiguousarray(wp).ravel(), "align_hwc_to_128": wc != 64}]
    layers = [{"type": "BinConv2D", "name": "bc", "input": "data", "weight": "w", "output": "cnt", "pads": list(pads),
               "strides": list(stride), "dilations": [1, 1]}]
    return df.write_model(layers, inits, [("data", [1, 12, 12, c])])


def test_weight_tensors_must_fit_their_layer(net):
    net.check_model(_binconv_model())
    with pytest.raises(RuntimeError, match="input channels"):
        net.check_model(_binconv_model(c=256, wc=128))  # the kernel would walk 36 words per filter, the tensor has 18
    with pytest.raises(RuntimeError, match="words per filter"):
        net.check_model(_binconv_model(words=10))  # a short weight tensor
    with pytest.raises(RuntimeError, match="words per filter"):
        net.check_model(_binconv_model(words=40))  # more words than the padded row
    with pytest.raises(RuntimeError, match="strides must be positive"):
        net.check_model(_binconv_model(stride=(0, 0)))  # a division by zero in the reference's shape inference
    with pytest.raises(RuntimeError, match="symmetric"):
        net.check_model(_binconv_model(pads=(1, 1, 2, 1)))  # dabnn/net.cpp:174-185
    with pytest.raises(RuntimeError, match="larger than its padded input"):
        net.check_model(_binconv_model(k=5, pads=(0, 0, 0, 0), c=64, wc=64, cout=8) if False else
                        df.write_model([{"type": "MaxPool", "name": "p", "input": "data", "output": "o",
                                         "kernel_shape": [20, 20], "pads": [0] * 4, "strides": [1, 1]}], [],
                                       [("data", [1, 12, 12, 64])]))


def test_float_layers_are_checked_too(net):
    r = np.random.default_rng(6)
    w = r.standard_normal((8, 3, 3, 4)).astype(np.float32)
    conv = {"type": "FpConv2D", "name": "c", "input": "data", "weight": "w", "output": "o", "pads": [1] * 4,
            "strides": [1, 1], "dilations": [1, 1]}
    ok = [{"name": "w", "shape": [8, 3, 3, 4], "data": w, "align_hwc_to_128": False}]
    net.check_model(df.write_model([conv], ok, [("data", [1, 8, 8, 4])]))
    with pytest.raises(RuntimeError, match="input channels"):
        net.check_model(df.write_model([conv], ok, [("data", [1, 8, 8, 3])]))
    with pytest.raises(RuntimeError, match="does not match its shape"):
        short = [{"name": "w", "shape": [8, 3, 3, 4], "data": w.ravel()[:100], "align_hwc_to_128": False}]
        net.check_model(df.write_model([conv], short, [("data", [1, 8, 8, 4])]))
    bias = dict(conv, bias="b")
    with pytest.raises(RuntimeError, match="bias b must hold 8 floats"):
        net.check_model(df.write_model([bias], ok + [{"name": "b", "shape": [5], "data": np.zeros(5, np.float32),
                                                       "align_hwc_to_128": False}], [("data", [1, 8, 8, 4])]))
    aff = {"type": "Affine", "name": "a", "input": "o", "a": "ka", "b": "kb", "output": "o2"}
    coef = lambda n, k: {"name": n, "shape": [k], "data": np.ones(k, np.float32), "align_hwc_to_128": False}
    net.check_model(df.write_model([conv, aff], ok + [coef("ka", 8), coef("kb", 8)], [("data", [1, 8, 8, 4])]))
    with pytest.raises(RuntimeError, match="coefficient kb must hold 8 floats"):
        net.check_model(df.write_model([conv, aff], ok + [coef("ka", 8), coef("kb", 7)], [("data", [1, 8, 8, 4])]))
    with pytest.raises(KeyError):
        net.check_model(df.write_model([dict(conv, input="nope")], ok, [("data", [1, 8, 8, 4])]))


def test_version_and_unsupported_layers(net):
    layers, inits, inputs = small()
    with pytest.raises(RuntimeError, match="model version should be 2"):
        net.check_model(df.write_model(layers, inits, inputs, version=1))
    bad = layers + [{"type": "Softmax", "name": "sm", "input": "logits", "output": "prob"}]
    with pytest.raises(RuntimeError, match="Not supported op Softmax"):
        net.check_model(df.write_model(bad, inits, inputs))


def test_split_and_shuffle_want_bit_blobs(net):
    """dabnn/layers/Split.h:19-23, Shuffle.h:16-20: only Bit blobs of 128, 256, 384 or 512 channels."""
    words = np.arange(2 * 4 * 4 * 4, dtype=np.uint64)
    bit = [{"name": "bits", "shape": [2, 4, 4, 256], "data": words, "data_type": "bit", "align_hwc_to_128": False}]
    net.check_model(df.write_model([{"type": "Shuffle", "name": "sh", "input": "bits", "output": "s"},
                                    {"type": "Split", "name": "sp", "input": "s", "outputs": ["l", "r"]}], bit,
                                   [("data", [1, 4, 4, 128])]))
    with pytest.raises(RuntimeError, match="Shuffle only supports bit mat"):
        net.check_model(df.write_model([{"type": "Shuffle", "name": "sh", "input": "data", "output": "s"}], [],
                                       [("data", [1, 4, 4, 128])]))
    with pytest.raises(RuntimeError, match="Split only supports bit mat"):
        net.check_model(df.write_model([{"type": "Split", "name": "sp", "input": "data", "outputs": ["l", "r"]}], [],
                                       [("data", [1, 4, 4, 128])]))


def test_a_layer_output_must_be_a_new_name(net):
    """A layer that makes a blob (convolution, pool, concat, split) may not name it like a blob that exists: the net
    would keep the existing blob, of another size, and the layer's kernel would write past it.  Checked on the host
    only; such a model never reaches a device."""
    layers, inits, inputs = small()
    net.check_model(df.write_model(layers, inits, inputs))
    convs = [i for i, l in enumerate(layers) if l["type"] in ("FpConv2D", "BinConv2D")]
    binconvs = [i for i, l in enumerate(layers) if l["type"] == "BinConv2D"]
    assert convs and binconvs

    def renamed(index, new_name):
        """layers with the output of layer `index` renamed, its readers following the new name."""
        old = layers[index]["output"]
        out = []
        for i, l in enumerate(layers):
            l = dict(l)
            if i == index:
                l["output"] = new_name
            elif i > index:
                for key in ("input", "input1", "input2"):
                    if l.get(key) == old:
                        l[key] = new_name
            out.append(l)
        return out

    # a convolution's output named like the net's input
    with pytest.raises(RuntimeError, match="already exists"):
        net.check_model(df.write_model(renamed(convs[0], inputs[0][0]), inits, inputs))
    # a BinConv's output named like an initializer (its own weight)
    bc = binconvs[0]
    with pytest.raises(RuntimeError, match="already exists"):
        net.check_model(df.write_model(renamed(bc, layers[bc]["weight"]), inits, inputs))
    # two BinConvs with the same output name would share the scratch blobs binaized_for_<out>_cal / col_for_<out>_cal
    if len(binconvs) > 1:
        with pytest.raises(RuntimeError, match="already exists"):
            net.check_model(df.write_model(renamed(binconvs[1], layers[bc]["output"]), inits, inputs))
    # an in-place layer re-pointing the input's name at another blob
    inplace = [i for i, l in enumerate(layers) if l["type"] in ("Affine", "Relu", "Add")]
    with pytest.raises(RuntimeError, match="already exists"):
        net.check_model(df.write_model(renamed(inplace[-1], inputs[0][0]), inits, inputs))
    # a later output named like a BinConv's scratch blob
    pool = {"type": "MaxPool", "name": "late", "input": inputs[0][0], "output": "col_for_%s_cal" % layers[bc]["output"],
            "kernel_shape": [2, 2], "pads": [0] * 4, "strides": [2, 2]}
    with pytest.raises(RuntimeError, match="already exists"):
        net.check_model(df.write_model(layers + [pool], inits, inputs))


def test_window_extents_are_bounded(net):
    """Kernel extents and output sizes that would overflow the int fields of the runtime are refused on the host."""
    with pytest.raises(RuntimeError, match="too large"):
        net.check_model(df.write_model([{"type": "MaxPool", "name": "p", "input": "data", "output": "o",
                                         "kernel_shape": [1 << 16, 1], "pads": [32767, 0, 32767, 0], "strides": [1, 1]}], [],
                                       [("data", [1, 12, 12, 64])]))
    w = np.zeros((1 << 10, 1, 1, 4), np.float32)
    conv = {"type": "FpConv2D", "name": "c", "input": "data", "weight": "w", "output": "o", "pads": [0] * 4,
            "strides": [1, 1], "dilations": [1, 1]}
    with pytest.raises(RuntimeError, match="too large"):
        net.check_model(df.write_model([conv], [{"name": "w", "shape": list(w.shape), "data": w, "align_hwc_to_128": False}],
                                       [("data", [1, 2048, 2048, 4])]))
