"""The .dab writer/reader (no GPU): round trip and FlatBuffers layout rules."""
import struct

import numpy as np

from dabnn_amd import dab_format as df
from dabnn_amd import models


def test_roundtrip_bireal18():
    for stem in (False, True):
        layers, inits, inputs = models.bireal18(3, stem=stem)
        buf = df.write_model(layers, inits, inputs)
        m = df.read_model(buf)
        assert m["version"] == 2 and m["inputs"] == inputs
        assert [l["type"] for l in m["layers"]] == [l["type"] for l in layers]
        for a, b in zip(layers, m["layers"]):
            for k, v in a.items():
                assert b[k] == v, (a["name"], k)
        for a, b in zip(inits, m["initializers"]):
            assert (a["name"], a["shape"], a["align_hwc_to_128"]) == (b["name"], b["shape"], b["align_hwc_to_128"])
            assert np.array_equal(np.asarray(a["data"]).ravel(), b["data"])
        assert sum(l["type"] == "BinConv2D" for l in layers) == 16


def test_roundtrip_dense_net_with_concat_and_prelu():
    layers, inits, inputs = models.dense_bnn(4)
    m = df.read_model(df.write_model(layers, inits, inputs))
    assert [l["type"] for l in m["layers"]].count("Concat") == 5 and [l["type"] for l in m["layers"]].count("PRelu") == 2
    for a, b in zip(layers, m["layers"]):
        for k, v in a.items():
            assert b[k] == v, (a["name"], k)
    for a, b in zip(inits, m["initializers"]):
        assert (a["name"], a["shape"]) == (b["name"], b["shape"])
        assert np.array_equal(np.asarray(a["data"]).ravel(), b["data"])


def test_layout_rules():
    layers, inits, inputs = models.small_bnn(0)
    buf = df.write_model(layers, inits, inputs)
    root = struct.unpack_from("<I", buf, 0)[0]
    assert root % 4 == 0 and len(buf) % 8 == 0
    m = df.read_model(buf)
    base = np.frombuffer(buf, dtype=np.uint8).ctypes.data
    for t in m["initializers"]:
        off = t["data"].ctypes.data - base
        assert off % t["data"].itemsize == 0, t["name"]  # uint64 payloads on 8-byte, float on 4-byte boundaries
    # vtable of the root table: 4 fields -> 4 + 2*4 bytes
    vt = root - struct.unpack_from("<i", buf, root)[0]
    assert struct.unpack_from("<H", buf, vt)[0] == 12


def test_weight_packing_rule():
    w = np.ones((2, 3, 3, 64), dtype=np.float32)
    assert models.pack_weight(w).shape == (2, 9)
    w = np.ones((2, 3, 3, 192), dtype=np.float32)
    p = models.pack_weight(w)
    assert p.shape == (2, 28) and (p[:, :27] == 2**64 - 1).all() and (p[:, 27] == 0).all()
    import oracle as orc
    r = np.random.default_rng(0)
    for c in (64, 128, 192):
        wf = r.standard_normal((5, 3, 3, c)).astype(np.float32)
        np.testing.assert_array_equal(models.pack_weight(wf), orc.pack_weight(wf))
    s, b, m, v = (r.standard_normal(8).astype(np.float32) for _ in range(4))
    v = np.abs(v) + 0.5
    for k in (0, 576):
        a0, b0 = models.fold_bn(s, b, m, v, 1e-5, k)
        a1, b1 = orc.bn_fold(s, b, m, v, 1e-5, k)
        np.testing.assert_allclose(a0, a1, rtol=1e-6)
        np.testing.assert_allclose(b0, b1, rtol=1e-5, atol=1e-5)
