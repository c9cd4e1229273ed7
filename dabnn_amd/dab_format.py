"""Writer and reader for dabnn's ``.dab`` model files (FlatBuffers, schema
``common/dab.fbs`` of the reference, model version 2).

The flatbuffers package is not available here, so the wire format is produced
directly: a back-to-front builder that follows the FlatBuffers encoding rules
(little endian; tables with vtables of 16-bit field offsets; vectors and
strings as 32-bit length + payload; forward 32-bit offsets; scalars aligned to
their size).  Files written here load in the C++ ``bnn::Net`` of this package
and are laid out the way ``flatc``-generated code expects.

Field order (= vtable slot) of every table is the declaration order in
``common/dab.fbs``:
  Tensor  data_type, bin_data, float32_data, shape, name, align_hwc_to_128
  Input   shape, name
  Layer   type, fp_conv2d_param, bin_conv2d_param, avepool_param, maxpool_param,
          relu_param, softmax_param, fc_param, add_param, concat_param,
          affine_param, binarize_param, split_param, shuffle_param, name, prelu_param
  Model   layers, initializers, inputs, version
"""
import struct

import numpy as np

MODEL_VERSION = 2  # BNN_LATEST_MODEL_VERSION, common/macros.h:6

DATA_FLOAT32, DATA_BIT = 0, 1
LAYER_TYPES = ["FpConv2D", "AvePool", "MaxPool", "Relu", "Softmax", "FC", "Add", "Concat", "BinConv2D", "Affine",
               "Binarize", "Split", "Shuffle", "PRelu"]
LAYER_TYPE_ID = {n: i for i, n in enumerate(LAYER_TYPES)}
# Layer table: slot of the parameter table of each layer type
LAYER_PARAM_SLOT = {"FpConv2D": 1, "BinConv2D": 2, "AvePool": 3, "MaxPool": 4, "Relu": 5, "Softmax": 6, "FC": 7,
                    "Add": 8, "Concat": 9, "Affine": 10, "Binarize": 11, "Split": 12, "Shuffle": 13, "PRelu": 15}
LAYER_NAME_SLOT = 14

# parameter tables: ordered (field, kind); kind: s = string, iv = [int], sv = [string], i = int
PARAM_FIELDS = {
    "FpConv2D": [("input", "s"), ("weight", "s"), ("bias", "s"), ("pads", "iv"), ("strides", "iv"), ("dilations", "iv"),
                 ("output", "s")],
    "BinConv2D": [("input", "s"), ("weight", "s"), ("bias", "s"), ("pads", "iv"), ("strides", "iv"),
                  ("dilations", "iv"), ("output", "s")],
    "AvePool": [("input", "s"), ("kernel_shape", "iv"), ("pads", "iv"), ("strides", "iv"), ("output", "s")],
    "MaxPool": [("input", "s"), ("kernel_shape", "iv"), ("pads", "iv"), ("strides", "iv"), ("output", "s")],
    "Relu": [("input", "s"), ("output", "s")],
    "Softmax": [("input", "s"), ("output", "s")],
    "FC": [("input", "s"), ("weight", "s"), ("bias", "s"), ("output", "s")],
    "Add": [("input1", "s"), ("input2", "s"), ("output", "s")],
    "Concat": [("inputs", "sv"), ("axis", "i"), ("output", "s")],
    "Affine": [("input", "s"), ("a", "s"), ("b", "s"), ("output", "s")],
    "Binarize": [("input", "s"), ("output", "s")],
    "Split": [("input", "s"), ("outputs", "sv")],
    "Shuffle": [("input", "s"), ("output", "s")],
    "PRelu": [("input", "s"), ("slope", "s"), ("output", "s")],
}


class Builder:
    """Minimal FlatBuffers builder; the buffer grows towards lower addresses.

    Offsets handed out are distances from the END of the finished buffer, as in
    the official builders."""

    def __init__(self, trim_vtables=False):
        self.trim_vtables = trim_vtables  # drop trailing absent slots from every vtable, as flatc's builders do
        self.chunks = []  # in prepend order
        self.size = 0
        self.minalign = 1
        self.vtables = {}  # bytes -> offset, for vtable sharing

    def _prepend(self, b):
        self.chunks.append(bytes(b))
        self.size += len(b)

    def _pad(self, n):
        if n:
            self._prepend(b"\x00" * n)

    def prep(self, align, additional):
        """Pad so that after `additional` more bytes the write position is `align`-aligned."""
        self.minalign = max(self.minalign, align)
        self._pad((-(self.size + additional)) % align)

    def string(self, s):
        data = s.encode("utf-8")
        self.prep(4, len(data) + 1)
        self._prepend(data + b"\x00")
        self._prepend(struct.pack("<I", len(data)))
        return self.size

    def vector_scalars(self, arr, fmt_align):
        """arr: numpy array of a little-endian scalar dtype."""
        data = np.ascontiguousarray(arr).tobytes()
        self.prep(4, len(data))
        self.prep(fmt_align, len(data))
        self._prepend(data)
        self._prepend(struct.pack("<I", len(arr)))
        return self.size

    def vector_offsets(self, offsets):
        self.prep(4, 4 * len(offsets))
        for off in reversed(offsets):
            # the slot written now ends up at distance size+4 from the end; it points forward to `off`
            self._prepend(struct.pack("<I", self.size + 4 - off))
        self._prepend(struct.pack("<I", len(offsets)))
        return self.size

    def table(self, n_slots, fields):
        """fields: list of (slot, kind, value); kind in {'off', 'u8', 'i8', 'i32', 'u32', 'bool'}."""
        table_end = self.size
        positions = {}
        # larger scalars first is customary; any order is valid
        for slot, kind, value in sorted(fields, key=lambda f: -{"off": 4, "i32": 4, "u32": 4}.get(f[1], 1)):
            if kind == "off":
                self.prep(4, 0)
                self._prepend(struct.pack("<I", self.size + 4 - value))
            elif kind in ("i32", "u32"):
                self.prep(4, 0)
                self._prepend(struct.pack("<i" if kind == "i32" else "<I", value))
            else:
                self._prepend(struct.pack("<b" if kind == "i8" else "<B", int(value)))
            positions[slot] = self.size
        self.prep(4, 0)
        self._prepend(b"\x00\x00\x00\x00")  # soffset to the vtable, patched below
        table_off = self.size
        vt = [4 + 2 * n_slots, table_off - table_end]
        for slot in range(n_slots):
            vt.append(table_off - positions[slot] if slot in positions else 0)
        if self.trim_vtables:
            while len(vt) > 2 and vt[-1] == 0:
                vt.pop()
            vt[0] = 2 * len(vt)
        vt_bytes = struct.pack("<%dH" % len(vt), *vt)
        if vt_bytes in self.vtables:
            vt_off = self.vtables[vt_bytes]
        else:
            self.prep(2, len(vt_bytes))
            self._prepend(vt_bytes)
            vt_off = self.size
            self.vtables[vt_bytes] = vt_off
        # soffset = table position - vtable position (positions measured from the start: larger offset = earlier)
        self._patch(table_off, struct.pack("<i", vt_off - table_off))
        return table_off

    def _patch(self, off_from_end, data):
        # find the chunk that starts at distance off_from_end from the end
        pos = 0
        for i, ch in enumerate(self.chunks):
            pos += len(ch)
            if pos == off_from_end:
                assert len(ch) >= len(data)
                self.chunks[i] = data + ch[len(data):]
                return
        raise AssertionError("patch position not on a chunk boundary")

    def finish(self, root):
        self.prep(self.minalign, 4)
        self._prepend(struct.pack("<I", self.size + 4 - root))
        return b"".join(reversed(self.chunks))


def _param_table(b, ltype, params):
    fields = []
    spec = PARAM_FIELDS[ltype]
    # children first
    built = {}
    for name, kind in spec:
        if name not in params or params[name] is None:
            continue
        v = params[name]
        if kind == "s":
            built[name] = b.string(v)
        elif kind == "iv":
            built[name] = b.vector_scalars(np.asarray(v, dtype="<i4"), 4)
        elif kind == "sv":
            built[name] = b.vector_offsets([b.string(s) for s in v])
    for slot, (name, kind) in enumerate(spec):
        if name in built:
            fields.append((slot, "off", built[name]))
        elif kind == "i" and name in params:
            fields.append((slot, "i32", int(params[name])))
    return b.table(len(spec), fields)


def write_model(layers, initializers, inputs, version=MODEL_VERSION, trim_vtables=False):
    """layers: list of dicts {"type": str, "name": str, **params};
    initializers: list of dicts {"name", "shape", "data" (np.float32 or np.uint64 array), "align_hwc_to_128": bool};
    inputs: list of (name, shape).  Returns the file content.  Scalars at their default (Float32 data, FpConv2D
    type, align_hwc_to_128 false) are left out and equal vtables are shared, as flatc's builders do; trim_vtables
    also drops the trailing absent slots of every vtable, their other habit."""
    b = Builder(trim_vtables)
    layer_offs = []
    for layer in layers:
        ltype = layer["type"]
        params = {k: v for k, v in layer.items() if k not in ("type", "name")}
        p_off = _param_table(b, ltype, params)
        fields = [(LAYER_PARAM_SLOT[ltype], "off", p_off)]
        if layer.get("name"):
            fields.append((LAYER_NAME_SLOT, "off", b.string(layer["name"])))
        if LAYER_TYPE_ID[ltype] != 0:
            fields.append((0, "i8", LAYER_TYPE_ID[ltype]))
        layer_offs.append(b.table(16, fields))
    init_offs = []
    for t in initializers:
        data = t["data"]
        name_off = b.string(t["name"])
        shape_off = b.vector_scalars(np.asarray(t["shape"], dtype="<u4"), 4)
        fields = [(3, "off", shape_off), (4, "off", name_off)]
        if data.dtype == np.uint64:
            fields.append((1, "off", b.vector_scalars(data.astype("<u8").ravel(), 8)))
            fields.append((0, "i8", DATA_BIT))
        else:
            fields.append((2, "off", b.vector_scalars(data.astype("<f4").ravel(), 4)))
        if t.get("align_hwc_to_128"):
            fields.append((5, "bool", 1))
        init_offs.append(b.table(6, fields))
    input_offs = []
    for name, shape in inputs:
        n_off = b.string(name)
        s_off = b.vector_scalars(np.asarray(shape, dtype="<u4"), 4)
        input_offs.append(b.table(2, [(0, "off", s_off), (1, "off", n_off)]))
    layers_v = b.vector_offsets(layer_offs)
    inits_v = b.vector_offsets(init_offs)
    inputs_v = b.vector_offsets(input_offs)
    root = b.table(4, [(0, "off", layers_v), (1, "off", inits_v), (2, "off", inputs_v), (3, "u32", version)])
    return b.finish(root)


# ---------------------------------------------------------------------------- reader
class _Table:
    def __init__(self, buf, pos):
        self.buf, self.pos = buf, pos
        self.vt = pos - struct.unpack_from("<i", buf, pos)[0]
        self.vt_size = struct.unpack_from("<H", buf, self.vt)[0]

    def _field(self, slot):
        o = 4 + 2 * slot
        if o >= self.vt_size:
            return 0
        return struct.unpack_from("<H", self.buf, self.vt + o)[0]

    def scalar(self, slot, fmt, default=0):
        f = self._field(slot)
        return struct.unpack_from(fmt, self.buf, self.pos + f)[0] if f else default

    def _indirect(self, slot):
        f = self._field(slot)
        if not f:
            return None
        p = self.pos + f
        return p + struct.unpack_from("<I", self.buf, p)[0]

    def string(self, slot):
        p = self._indirect(slot)
        if p is None:
            return None
        n = struct.unpack_from("<I", self.buf, p)[0]
        return bytes(self.buf[p + 4:p + 4 + n]).decode("utf-8")

    def vector(self, slot, dtype):
        p = self._indirect(slot)
        if p is None:
            return None
        n = struct.unpack_from("<I", self.buf, p)[0]
        return np.frombuffer(self.buf, dtype=dtype, count=n, offset=p + 4)

    def table(self, slot):
        p = self._indirect(slot)
        return None if p is None else _Table(self.buf, p)

    def vector_of(self, slot, kind):
        p = self._indirect(slot)
        if p is None:
            return None
        n = struct.unpack_from("<I", self.buf, p)[0]
        out = []
        for i in range(n):
            e = p + 4 + 4 * i
            t = e + struct.unpack_from("<I", self.buf, e)[0]
            if kind == "table":
                out.append(_Table(self.buf, t))
            else:
                ln = struct.unpack_from("<I", self.buf, t)[0]
                out.append(bytes(self.buf[t + 4:t + 4 + ln]).decode("utf-8"))
        return out


def read_model(buf):
    """Inverse of write_model (returns the same plain structures)."""
    buf = bytes(buf)
    root = _Table(buf, struct.unpack_from("<I", buf, 0)[0])
    model = {"version": root.scalar(3, "<I"), "layers": [], "initializers": [], "inputs": []}
    for t in root.vector_of(2, "table") or []:
        model["inputs"].append((t.string(1), [int(v) for v in t.vector(0, "<u4")]))
    for t in root.vector_of(1, "table") or []:
        dtype = t.scalar(0, "<b")
        data = t.vector(1, "<u8") if dtype == DATA_BIT else t.vector(2, "<f4")
        model["initializers"].append({"name": t.string(4), "shape": [int(v) for v in t.vector(3, "<u4")], "data": data,
                                      "align_hwc_to_128": bool(t.scalar(5, "<B"))})
    for t in root.vector_of(0, "table") or []:
        ltype = LAYER_TYPES[t.scalar(0, "<b")]
        layer = {"type": ltype, "name": t.string(LAYER_NAME_SLOT) or ""}
        p = t.table(LAYER_PARAM_SLOT[ltype])
        for slot, (name, kind) in enumerate(PARAM_FIELDS[ltype]):
            if kind == "s":
                v = p.string(slot)
            elif kind == "iv":
                v = p.vector(slot, "<i4")
                v = None if v is None else [int(x) for x in v]
            elif kind == "sv":
                v = p.vector_of(slot, "string")
            else:
                v = p.scalar(slot, "<i")
            if v is not None:
                layer[name] = v
        model["layers"].append(layer)
    return model
