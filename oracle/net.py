"""CPU restatement of the reference's layer loop (dabnn/net.cpp:140-286) on
top of the oracle kernels.  Test infrastructure only.

Takes the plain model description used by ``dabnn_amd.dab_format`` (layers,
initializers, inputs) and one NHWC image; returns every blob by name.  Affine,
Add and Relu work in place and their output name aliases the input blob, as
ADD_INPLACE_LAYER does (common/flatbuffers_helper.h:68-73); BinConv follows
the x86 dispatch (dabnn/layers/BinConv.cpp:80-98) via orc.binconv_forward.
"""
import numpy as np

import oracle as orc


def run_model(layers, initializers, x, record=None):
    """x: float32 [H, W, C].  record: optional dict that receives a copy of each BinConv's raw counts."""
    blobs = {t["name"]: t for t in initializers}
    act = {"data": np.ascontiguousarray(x, dtype=np.float32)}

    def weights(name):
        t = blobs[name]
        return np.asarray(t["data"]), t["shape"]

    for layer in layers:
        ty = layer["type"]
        if ty in ("FpConv2D", "BinConv2D"):
            src = act[layer["input"]]
            w, shape = weights(layer["weight"])
            cout, kh, kw, cin = shape
            pad_h, pad_w = layer["pads"][0], layer["pads"][1]
            sh, sw = layer["strides"][0], layer["strides"][1]
            if ty == "BinConv2D":
                wp = w.reshape(cout, -1)
                if cin == 64 and (kh, kw) != (3, 3):
                    out = orc.baseline_bconv(orc.pack_mat(src), wp, kh, kw, pad_h, pad_w, sh, sw)
                else:
                    out, _ = orc.binconv_forward(src, wp, kh, kw, pad_h, pad_w, sh, sw)
                if record is not None:
                    record[layer["output"]] = out.copy()
            else:
                bias = np.asarray(blobs[layer["bias"]]["data"]) if layer.get("bias") else None
                out = orc.fconv(src, w.reshape(cout, kh, kw, cin), bias, kh, kw, pad_h, pad_w, sh, sw)
            act[layer["output"]] = out
        elif ty == "Affine":
            buf = act[layer["input"]]
            orc.affine_inplace(buf, np.asarray(blobs[layer["a"]]["data"]), np.asarray(blobs[layer["b"]]["data"]))
            act[layer["output"]] = buf
        elif ty == "Add":
            buf = act[layer["input1"]]
            orc.add_inplace(buf, act[layer["input2"]])
            act[layer["output"]] = buf
        elif ty == "Relu":
            buf = act[layer["input"]]
            np.maximum(buf, 0, out=buf)
            act[layer["output"]] = buf
        elif ty in ("MaxPool", "AvePool"):
            src = act[layer["input"]]
            kh, kw = layer["kernel_shape"]
            fn = orc.max_pool if ty == "MaxPool" else orc.ave_pool
            act[layer["output"]] = fn(src, kh, kw, layer["pads"][0], layer["pads"][1], layer["strides"][0],
                                      layer["strides"][1])
        else:
            raise RuntimeError("Not supported op " + ty)
    return act
