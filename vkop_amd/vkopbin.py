"""The `.vkopbin` model file: reader and writer.

Layout (little endian; writer model/pypi/onnx2vkop/dag.py:102-217, reader
model/load.cpp:98-285 and model/load.hpp:163-275):

  shapes   = u32 count, then per entry: string name, dims
  string   = u32 length, bytes (utf-8)
  dims     = u32 count, u32 each
  file     = shapes inputs, shapes outputs,
             u32 nodes, per node: string op_type, string name, dict attributes,
                 shapes inputs, shapes outputs, u32 + strings dependencies,
                 u32 + strings dependents,
             u32 initializers, per entry: string name, string dtype, dims,
                 u64 byte length, bytes,
             u32 levels, per level: u32 + strings node names
  dict     = u32 count, per entry: string key, u8 tag, value:
                 0 string, 1 i64, 2 f32, 3 list of u32, 4 list of f32

The reader gives attribute values the textual form the C++ reader gives them
(std::to_string of the number; lists as "[a, b]"), since operators parse them
from text (ops/Softmax.hpp:25-40, ops/Topk.hpp:31-44).  Every length is checked
against the end of the file; a short or malformed file raises ValueError.
"""
import struct

import numpy as np

DTYPES = {"float32": np.float32, "uint8": np.uint8, "int8": np.int8, "uint16": np.uint16, "int16": np.int16,
          "int32": np.int32, "int64": np.int64, "bool": np.bool_, "float16": np.float16, "float64": np.float64,
          "uint32": np.uint32, "uint64": np.uint64}


class _Cursor:
    def __init__(self, data):
        self.data, self.at = memoryview(data), 0

    def take(self, n, what):
        if n < 0 or self.at + n > len(self.data):
            raise ValueError(f"unexpected end of file in {what} at byte {self.at}")
        out = self.data[self.at:self.at + n]
        self.at += n
        return out

    def u32(self, what="u32"):
        return struct.unpack("<I", self.take(4, what))[0]

    def string(self):
        return bytes(self.take(self.u32("string length"), "string")).decode("utf-8")

    def dims(self):
        return [self.u32("dim") for _ in range(self.u32("dims count"))]

    def shapes(self):
        return [{"name": self.string(), "shape": self.dims()} for _ in range(self.u32("shapes count"))]

    def strings(self):
        return [self.string() for _ in range(self.u32("names count"))]


def _f32_text(v):
    return f"{v:.6f}"  # std::to_string(float)


def _read_dict(c):
    out = {}
    for _ in range(c.u32("attribute count")):
        key = c.string()
        tag = c.take(1, "attribute tag")[0]
        if tag == 0:
            out[key] = c.string()
        elif tag == 1:
            out[key] = str(struct.unpack("<q", c.take(8, "i64 attribute"))[0])
        elif tag == 2:
            out[key] = _f32_text(struct.unpack("<f", c.take(4, "f32 attribute"))[0])
        elif tag == 3:
            out[key] = "[" + ", ".join(str(c.u32()) for _ in range(c.u32("list length"))) + "]"
        elif tag == 4:
            n = c.u32("list length")
            out[key] = "[" + ", ".join(_f32_text(struct.unpack("<f", c.take(4, "f32 list"))[0]) for _ in range(n)) + "]"
        else:
            raise ValueError(f"unknown attribute type tag {tag} for {key!r}")   # model/load.hpp:256-258
    return out


def read_model(path_or_bytes):
    """-> dict(inputs, outputs, nodes, initializers, levels); initializers map name -> numpy array."""
    data = path_or_bytes if isinstance(path_or_bytes, (bytes, bytearray)) else open(path_or_bytes, "rb").read()
    c = _Cursor(data)
    model = {"inputs": c.shapes(), "outputs": c.shapes(), "nodes": [], "initializers": {}, "levels": []}
    for _ in range(c.u32("node count")):
        node = {"op_type": c.string(), "name": c.string()}
        node["attributes"] = _read_dict(c)
        node["inputs"], node["outputs"] = c.shapes(), c.shapes()
        node["dependencies"], node["dependents"] = c.strings(), c.strings()
        model["nodes"].append(node)
    for _ in range(c.u32("initializer count")):
        name, dtype, dims = c.string(), c.string(), c.dims()
        size = struct.unpack("<Q", c.take(8, "initializer length"))[0]
        raw = bytes(c.take(size, f"initializer {name!r}"))
        if dtype not in DTYPES:
            raise ValueError(f"initializer {name!r}: unsupported dtype {dtype!r}")
        arr = np.frombuffer(raw, dtype=DTYPES[dtype])
        model["initializers"][name] = arr.reshape(dims) if int(np.prod(dims, dtype=np.int64)) == arr.size else arr
    model["levels"] = [c.strings() for _ in range(c.u32("level count"))]
    return model


def _w_string(out, s):
    b = s.encode("utf-8")
    out += struct.pack("<I", len(b)) + b


def _w_shapes(out, shapes):
    out += struct.pack("<I", len(shapes))
    for s in shapes:
        _w_string(out, s["name"])
        out += struct.pack("<I", len(s["shape"])) + b"".join(struct.pack("<I", int(d)) for d in s["shape"])


def _w_strings(out, names):
    out += struct.pack("<I", len(names))
    for n in names:
        _w_string(out, n)


def _w_dict(out, d):
    out += struct.pack("<I", len(d))
    for key, v in d.items():
        _w_string(out, key)
        if isinstance(v, str):
            out += b"\x00"
            _w_string(out, v)
        elif isinstance(v, bool) or isinstance(v, (int, np.integer)):
            out += b"\x01" + struct.pack("<q", int(v))
        elif isinstance(v, (float, np.floating)):
            out += b"\x02" + struct.pack("<f", float(v))
        elif isinstance(v, (list, tuple)) and all(isinstance(e, (int, np.integer)) for e in v):
            out += b"\x03" + struct.pack("<I", len(v)) + b"".join(struct.pack("<I", int(e)) for e in v)
        elif isinstance(v, (list, tuple)) and all(isinstance(e, (float, np.floating)) for e in v):
            out += b"\x04" + struct.pack("<I", len(v)) + b"".join(struct.pack("<f", float(e)) for e in v)
        else:
            raise ValueError(f"unsupported attribute {key!r}: {v!r}")


def levels_of(nodes):
    """Nodes grouped so that each comes after all it depends on (Kahn's algorithm by generations,
    model/pypi/onnx2vkop/dag.py:62-100)."""
    left = {n["name"]: set(n.get("dependencies", [])) for n in nodes}
    levels = []
    while left:
        ready = [name for name, deps in left.items() if not deps]
        if not ready:
            raise ValueError("dependency cycle among nodes")
        levels.append(ready)
        for name in ready:
            del left[name]
        for deps in left.values():
            deps.difference_update(ready)
    return levels


def write_model(inputs, outputs, nodes, initializers=None, levels=None):
    """-> bytes.  nodes: dicts with op_type, name, attributes, inputs, outputs and, optionally,
    dependencies/dependents (derived from the tensor names when absent)."""
    nodes = [dict(n) for n in nodes]
    producer = {o["name"]: n["name"] for n in nodes for o in n["outputs"]}
    for n in nodes:
        if "dependencies" not in n:
            n["dependencies"] = sorted({producer[i["name"]] for i in n["inputs"] if i["name"] in producer})
    for n in nodes:
        if "dependents" not in n:
            n["dependents"] = sorted(m["name"] for m in nodes if n["name"] in m["dependencies"])
    out = bytearray()
    _w_shapes(out, inputs)
    _w_shapes(out, outputs)
    out += struct.pack("<I", len(nodes))
    for n in nodes:
        _w_string(out, n["op_type"])
        _w_string(out, n["name"])
        _w_dict(out, n.get("attributes", {}))
        _w_shapes(out, n["inputs"])
        _w_shapes(out, n["outputs"])
        _w_strings(out, n["dependencies"])
        _w_strings(out, n["dependents"])
    initializers = initializers or {}
    out += struct.pack("<I", len(initializers))
    names = {v: k for k, v in DTYPES.items()}
    for name, arr in initializers.items():
        arr = np.ascontiguousarray(arr)
        _w_string(out, name)
        _w_string(out, names[arr.dtype.type])
        out += struct.pack("<I", arr.ndim) + b"".join(struct.pack("<I", d) for d in arr.shape)
        out += struct.pack("<Q", arr.nbytes) + arr.tobytes()
    levels = levels_of(nodes) if levels is None else levels
    out += struct.pack("<I", len(levels))
    for level in levels:
        _w_strings(out, level)
    return bytes(out)
