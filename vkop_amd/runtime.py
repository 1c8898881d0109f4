"""Runs the nodes of a `.vkopbin` model (vkop_amd.vkopbin.read_model) on the GPU operators.

The Python counterpart of the C++ Runtime::LoadModel/Run pair
(vkop_amd/host/include/core/Runtime.hpp; reference core/runtime.cpp:33-363,404-458):
nodes run level by level in the file's order; a TopK that alone reads the
output of a Softmax along the same axis, where that output is no model output,
runs as the fused operator, and so does a Reduce "max" over that one axis.  A
node of any other kind than Softmax, TopK, Reduce ("max", one axis) and Nms
raises NotImplementedError naming it.
"""
from . import ops


def _axis(text, rank):
    a = int(text)
    return a + rank if a < 0 else a


def _axes(node):
    text = node["attributes"].get("axes", "[]").strip("[] ")
    return [int(v) for v in text.split(",")] if text else []


def plan(model, fuse=True):
    """-> list of (kind, node, source) in execution order; kind is 'softmax', 'topk', 'softmax_topk', 'reduce_max',
    'softmax_reduce_max' or 'nms'; source is the Softmax node a fused node reads through, else None."""
    by_name = {n["name"]: n for n in model["nodes"]}
    producer = {o["name"]: n for n in model["nodes"] for o in n["outputs"]}
    readers = {}
    for n in model["nodes"]:
        for i in n["inputs"]:
            readers[i["name"]] = readers.get(i["name"], 0) + 1
    outputs = {o["name"] for o in model["outputs"]}
    kinds = {"Softmax": "softmax", "TopK": "topk", "Nms": "nms", "Reduce": "reduce_max"}
    fused = {}
    for n in model["nodes"]:
        if n["op_type"] not in kinds:
            raise NotImplementedError(f"node {n['name']}: operator {n['op_type']} is not part of this library")
        if n["op_type"] == "Reduce" and (n["attributes"].get("reduce_op") != "max" or len(_axes(n)) != 1):
            raise NotImplementedError(f"node {n['name']}: Reduce is implemented for reduce_op \"max\" over one axis")
        if not fuse or n["op_type"] not in ("TopK", "Reduce"):
            continue
        src = producer.get(n["inputs"][0]["name"])
        if src is None or src["op_type"] != "Softmax":
            continue
        t = src["outputs"][0]
        rank = len(t["shape"])
        sa = _axis(src["attributes"].get("axis", src["attributes"].get("dim", "0")), rank)   # ops/Softmax.hpp: default 0
        if n["op_type"] == "Reduce":
            if rank < 2:
                continue
            ta = _axis(_axes(n)[0], rank)
        else:
            ta = _axis(n["attributes"].get("axis", "-1"), rank)                              # ops/Topk.hpp:41
        if readers.get(t["name"], 0) == 1 and t["name"] not in outputs and (rank == 1 or sa == ta):
            fused[n["name"]] = src
    skipped = {s["name"] for s in fused.values()}
    steps = []
    for level in model["levels"]:
        for name in level:
            n = by_name[name]
            if name in skipped:
                continue
            if name in fused:
                steps.append(("softmax_topk" if n["op_type"] == "TopK" else "softmax_reduce_max", n, fused[name]))
            else:
                steps.append((kinds[n["op_type"]], n, None))
    return steps


def run_model(model, inputs, fuse=True):
    """inputs: name -> device tensor.  -> dict of the model's outputs (device tensors)."""
    tensors = dict(inputs)
    for name, arr in model["initializers"].items():
        tensors.setdefault(name, arr)      # host arrays: only attributes-in-disguise (TopK's K) are read
    for kind, n, src in plan(model, fuse):
        a = n["attributes"]
        outs = [o["name"] for o in n["outputs"]]
        if kind == "softmax":
            x = tensors[n["inputs"][0]["name"]]
            tensors[outs[0]] = ops.softmax(x, _axis(a.get("axis", a.get("dim", "0")), x.dim()))
            continue
        if kind in ("reduce_max", "softmax_reduce_max"):
            x = tensors[(src or n)["inputs"][0]["name"]]
            ax = _axis(_axes(n)[0], x.dim())
            y = ops.softmax_reduce_max(x, ax) if src else ops.reduce_max(x, ax)
            tensors[outs[0]] = y.unsqueeze(ax) if int(a.get("keepdims", "1")) == 1 else y          # ops/Reduce.hpp:152
            continue
        if kind == "nms":
            rec, _ = ops.nms(tensors[n["inputs"][0]["name"]], tensors[n["inputs"][1]["name"]], float(a.get("iou_threshold", 0)),
                             float(a.get("score_threshold", 0)), int(a.get("max_output_boxes_per_class", 0)),
                             int(a.get("center_point_box", 0)))
            tensors[outs[0]] = rec
            continue
        k = a.get("K", a.get("k"))
        if k is None and len(n["inputs"]) > 1:      # ONNX keeps K in the second input
            k = int(tensors[n["inputs"][1]["name"]].reshape(-1)[0])
        k = int(k) if k is not None else 1          # ops/Topk.hpp:40
        largest = int(a.get("largest", "1")) != 0
        if kind == "softmax_topk":
            x = tensors[src["inputs"][0]["name"]]
            v, i = ops.softmax_topk(x, k, _axis(a.get("axis", "-1"), x.dim()), largest)
        else:
            x = tensors[n["inputs"][0]["name"]]
            v, i = ops.topk(x, k, _axis(a.get("axis", "-1"), x.dim()), largest, int(a.get("sorted", "1")) != 0)
        tensors[outs[0]], tensors[outs[1]] = v, i
    return {o["name"]: tensors[o["name"]] for o in model["outputs"]}
