"""CPU restatement of the reference's layer loop (dabnn/net.cpp:140-286) on
top of the oracle kernels.  Test infrastructure only.

Takes the plain model description used by ``dabnn_amd.dab_format`` (layers,
initializers, inputs) and one NHWC image; returns every blob by name.  Affine,
Add, Relu and PRelu work in place and their output name aliases the input blob, as
ADD_INPLACE_LAYER does (common/flatbuffers_helper.h:68-73); BinConv follows
the x86 dispatch (dabnn/layers/BinConv.cpp:80-98) via orc.binconv_forward.
"""
import numpy as np

import oracle as orc


def _apply(layer, act, blobs, record=None):
    """Runs one layer on the activations in ``act`` (in-place layers alias their output name to the input array)."""
    def weights(name):
        t = blobs[name]
        return np.asarray(t["data"]), t["shape"]

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
        orc.relu_inplace(buf)
        act[layer["output"]] = buf
    elif ty == "PRelu":
        buf = act[layer["input"]]
        orc.prelu_inplace(buf, np.asarray(blobs[layer["slope"]]["data"]))
        act[layer["output"]] = buf
    elif ty == "Concat":
        assert layer["axis"] == 3 and len(layer["inputs"]) == 2  # dabnn/net.cpp:230-236
        act[layer["output"]] = orc.concat(act[layer["inputs"][0]], act[layer["inputs"][1]])
    elif ty in ("MaxPool", "AvePool"):
        src = act[layer["input"]]
        kh, kw = layer["kernel_shape"]
        fn = orc.max_pool if ty == "MaxPool" else orc.ave_pool
        act[layer["output"]] = fn(src, kh, kw, layer["pads"][0], layer["pads"][1], layer["strides"][0],
                                  layer["strides"][1])
    elif ty == "Split":  # dabnn/net.cpp:245-250
        o1, o2 = orc.split_bit(act[layer["input"]])
        act[layer["outputs"][0]], act[layer["outputs"][1]] = o1, o2
    elif ty == "Shuffle":  # dabnn/net.cpp:251-256, in place
        buf = act[layer["input"]]
        if buf.dtype != np.uint64:
            raise RuntimeError("Shuffle only supports bit mat")
        orc.shuffle_bit(buf)
        act[layer["output"]] = buf
    else:
        raise RuntimeError("Not supported op " + ty)


def run_model(layers, initializers, x, record=None):
    """x: float32 [H, W, C].  record: optional dict that receives a copy of each BinConv's raw counts."""
    blobs = {t["name"]: t for t in initializers}
    act = {"data": np.ascontiguousarray(x, dtype=np.float32)}
    for layer in layers:
        _apply(layer, act, blobs, record)
    return act


_INPLACE = {"Affine": "input", "Add": "input1", "Relu": "input", "PRelu": "input"}


def run_segments(layers, initializers, fetch, absent=()):
    """Layer-by-layer check with the other implementation's own activations as inputs.

    A sign network amplifies a one-ulp difference in a float layer into flipped bits downstream, so two correct
    implementations drift apart end to end.  Here the layers are cut into segments (a layer that writes a new blob
    plus the in-place layers that later rewrite that blob); every segment is evaluated on the CPU from ``fetch(name)`` -- the
    final content of the input blobs as the implementation under test holds them after its run -- and yields
    (output blob name, type of the first layer, CPU result).  Valid when a blob is only read after the in-place layers
    on it have run, which holds for the graphs the converter emits (tools/onnx2bnn/OnnxConverter.cpp:583-639).
    ``absent`` names blobs the implementation under test does not hold (it ran their producer and their one reader as
    one pass): the reader's segment then continues the producer's instead of starting from a fetched blob.
    """
    blobs = {t["name"]: t for t in initializers}
    root = {}

    def r(name):
        while name in root:
            name = root[name]
        return name

    segs, owner = [], {}
    for layer in layers:
        key = _INPLACE.get(layer["type"])
        if key is not None and r(layer[key]) in owner:
            owner[r(layer[key])].append(layer)  # joins the segment of the blob it rewrites, wherever that started
        elif key is None and "input" in layer and r(layer["input"]) in absent and r(layer["input"]) in owner:
            owner[r(layer["input"])].append(layer)  # reads a blob that only exists inside the other implementation's pass
            owner[layer["output"]] = owner[r(layer["input"])]
        else:
            segs.append([layer])
            owner[r(layer[key]) if key is not None else layer["output"]] = segs[-1]
        if key is not None:
            root[layer["output"]] = layer[key]
    for seg in segs:
        act = {}
        first = seg[0]
        for name in [first[key] for key in ("input", "input1", "input2") if key in first] + list(first.get("inputs", [])):
            act[name] = np.array(fetch(r(name)), dtype=np.float32, copy=True)
        for layer in seg:
            if layer is not first and layer["type"] == "Add":
                act[layer["input2"]] = np.array(fetch(r(layer["input2"])), dtype=np.float32, copy=True)
            _apply(layer, act, blobs)
        yield r(seg[-1]["output"]), first["type"], act[seg[-1]["output"]]


def time_images(job):
    """Worker of a process pool: runs ``reps`` images through run_model after one warm-up image, all workers starting
    at the wall-clock time ``start_at``; returns (reps, seconds).  job = (layers, initializers, reps, seed, start_at)."""
    import time
    layers, initializers, reps, seed, start_at = job
    x = np.random.default_rng(seed).standard_normal((224, 224, 3)).astype(np.float32)
    run_model(layers, initializers, x)
    while time.time() < start_at:
        time.sleep(0.001)
    t0 = time.perf_counter()
    for _ in range(reps):
        run_model(layers, initializers, x)
    return reps, time.perf_counter() - t0
