"""The .vkopbin model file: the Python reader against the reference's own model file
(model/add_conv_model.vkopbin, copied as a data fixture), writer -> reader round trips,
refusal of damaged files, and the execution plan built from a model."""
import os
import struct
import subprocess
import sys

import numpy as np
import pytest

from vkop_amd import runtime, vkopbin

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_reads_the_reference_converters_file():
    m = vkopbin.read_model(os.path.join(GOLDEN, "add_conv_model.vkopbin"))
    assert [i["name"] for i in m["inputs"]] == ["input_x1", "input_x2"] and m["inputs"][0]["shape"] == [1, 16, 8, 8]
    assert m["outputs"] == [{"name": "output", "shape": [1, 16, 8, 8]}]
    add, conv = m["nodes"]
    assert (add["op_type"], add["name"], add["attributes"], add["dependents"]) == ("Add", "node_add", {}, ["node_conv2d"])
    assert conv["attributes"] == {"group": "16", "pads": "[1, 1, 1, 1]", "auto_pad": "NOTSET", "strides": "[1, 1]",
                                  "dilations": "[1, 1]"}
    assert [i["name"] for i in conv["inputs"]] == ["add", "conv.weight", "conv.bias", "conv.weight_scale"]
    w = m["initializers"]["conv.weight"]
    assert w.dtype == np.int8 and w.shape == (16, 1, 3, 3) and w.ravel()[:4].tolist() == [39, 127, 61, 18]
    assert m["initializers"]["conv.bias"].dtype == np.float32 and m["initializers"]["conv.bias"].shape == (16,)
    assert m["levels"] == [["node_add"], ["node_conv2d"]]
    with pytest.raises(NotImplementedError, match="Add"):
        runtime.plan(m)


def test_writer_and_reader_round_trip_with_every_attribute_kind():
    nodes = [{"op_type": "Softmax", "name": "a", "attributes": {"axis": -1, "scale": 0.5, "note": "x", "l": [1, 2], "f": [0.25]},
              "inputs": [{"name": "in", "shape": [2, 3]}], "outputs": [{"name": "mid", "shape": [2, 3]}]},
             {"op_type": "TopK", "name": "b", "attributes": {"K": 2},
              "inputs": [{"name": "mid", "shape": [2, 3]}], "outputs": [{"name": "v", "shape": [2, 2]}, {"name": "i", "shape": [2, 2]}]}]
    init = {"w": np.arange(6, dtype=np.float16).reshape(2, 3), "k": np.array([2], dtype=np.int64)}
    data = vkopbin.write_model([{"name": "in", "shape": [2, 3]}], [{"name": "v", "shape": [2, 2]}, {"name": "i", "shape": [2, 2]}],
                               nodes, init)
    m = vkopbin.read_model(data)
    assert m["nodes"][0]["attributes"] == {"axis": "-1", "scale": "0.500000", "note": "x", "l": "[1, 2]", "f": "[0.250000]"}
    assert m["nodes"][1]["dependencies"] == ["a"] and m["nodes"][0]["dependents"] == ["b"]
    assert m["levels"] == [["a"], ["b"]]
    assert np.array_equal(m["initializers"]["w"], init["w"]) and m["initializers"]["k"].tolist() == [2]
    # the same bytes again from what was read (attributes as written)
    assert vkopbin.write_model(m["inputs"], m["outputs"], nodes, init) == data


def test_damaged_files_are_refused():
    data = open(os.path.join(GOLDEN, "classifier_head.vkopbin"), "rb").read()
    for n in range(len(data)):
        with pytest.raises(ValueError):
            vkopbin.read_model(data[:n])
    at = data.index(b"axis") + 4
    with pytest.raises(ValueError, match="tag"):
        vkopbin.read_model(data[:at] + b"\x09" + data[at + 1:])
    with pytest.raises(ValueError):
        vkopbin.read_model(struct.pack("<I", 0x7FFFFFFF) + data[4:])


def test_fixture_generator_reproduces_the_committed_files(tmp_path):
    names = ["classifier_head.vkopbin", "classifier_head_k_input.vkopbin", "detection_tail.vkopbin", "detection_chain.vkopbin", "two_heads.vkopbin"]
    before = {n: open(os.path.join(GOLDEN, n), "rb").read() for n in names}
    src = open(os.path.join(GOLDEN, "make_vkopbin.py")).read().replace("HERE = os.path.dirname(os.path.abspath(__file__))",
                                                                      f"HERE = {str(tmp_path)!r}")
    script = tmp_path / "make.py"
    script.write_text(src.replace("sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))",
                                  f"sys.path.insert(0, {os.path.dirname(os.path.dirname(GOLDEN))!r})"))
    subprocess.check_call([sys.executable, str(script)])
    for n in names:
        assert (tmp_path / n).read_bytes() == before[n]


def test_plan_fuses_only_a_private_softmax_along_the_same_axis():
    head = vkopbin.read_model(os.path.join(GOLDEN, "classifier_head.vkopbin"))
    assert [(k, n["name"]) for k, n, _ in runtime.plan(head)] == [("softmax_topk", "node_topk")]
    assert [(k, n["name"]) for k, n, _ in runtime.plan(head, fuse=False)] == [("softmax", "node_softmax"), ("topk", "node_topk")]
    shared = vkopbin.read_model(os.path.join(GOLDEN, "classifier_head_k_input.vkopbin"))     # probabilities are an output
    assert [k for k, _, _ in runtime.plan(shared)] == ["softmax", "topk"]
    other_axis = vkopbin.read_model(vkopbin.write_model(
        [{"name": "x", "shape": [4, 8]}], [{"name": "v", "shape": [4, 2]}, {"name": "i", "shape": [4, 2]}],
        [{"op_type": "Softmax", "name": "s", "attributes": {"axis": 0}, "inputs": [{"name": "x", "shape": [4, 8]}],
          "outputs": [{"name": "p", "shape": [4, 8]}]},
         {"op_type": "TopK", "name": "t", "attributes": {"K": 2, "axis": 1}, "inputs": [{"name": "p", "shape": [4, 8]}],
          "outputs": [{"name": "v", "shape": [4, 2]}, {"name": "i", "shape": [4, 2]}]}]))
    assert [k for k, _, _ in runtime.plan(other_axis)] == ["softmax", "topk"]


def test_plan_fuses_the_class_maximum_with_its_softmax():
    chain = vkopbin.read_model(os.path.join(GOLDEN, "detection_chain.vkopbin"))
    assert [(k, n["name"]) for k, n, _ in runtime.plan(chain)] == [("softmax_reduce_max", "node_max"), ("topk", "node_topk")]
    assert [k for k, _, _ in runtime.plan(chain, fuse=False)] == ["softmax", "reduce_max", "topk"]
    for attrs in ({"reduce_op": "sum", "axes": [1]}, {"reduce_op": "max", "axes": [0, 1]}):
        bad = vkopbin.read_model(vkopbin.write_model(
            [{"name": "x", "shape": [4, 8]}], [{"name": "y", "shape": [4]}],
            [{"op_type": "Reduce", "name": "r", "attributes": attrs, "inputs": [{"name": "x", "shape": [4, 8]}],
              "outputs": [{"name": "y", "shape": [4]}]}]))
        with pytest.raises(NotImplementedError, match="Reduce"):
            runtime.plan(bad)
    other_axis = vkopbin.read_model(vkopbin.write_model(
        [{"name": "x", "shape": [4, 8]}], [{"name": "y", "shape": [4]}],
        [{"op_type": "Softmax", "name": "s", "attributes": {"axis": 0}, "inputs": [{"name": "x", "shape": [4, 8]}],
          "outputs": [{"name": "p", "shape": [4, 8]}]},
         {"op_type": "Reduce", "name": "r", "attributes": {"reduce_op": "max", "axes": [1], "keepdims": 0},
          "inputs": [{"name": "p", "shape": [4, 8]}], "outputs": [{"name": "y", "shape": [4]}]}]))
    assert [k for k, _, _ in runtime.plan(other_axis)] == ["softmax", "reduce_max"]


def test_every_single_byte_change_parses_or_raises_value_error():
    for name in ("classifier_head.vkopbin", "detection_tail.vkopbin", "add_conv_model.vkopbin", "classifier_head_k_input.vkopbin"):
        data = open(os.path.join(GOLDEN, name), "rb").read()
        refused = 0
        for at in range(len(data)):
            for value in (0x00, 0x7F, 0xFF, data[at] ^ 1):
                if value == data[at]:
                    continue
                try:
                    vkopbin.read_model(data[:at] + bytes([value]) + data[at + 1:])
                except ValueError:
                    refused += 1
        assert refused > 100


def test_levels_with_two_nodes():
    two = vkopbin.read_model(os.path.join(GOLDEN, "two_heads.vkopbin"))
    assert two["levels"] == [["node_softmax", "node_nms"], ["node_topk"]]
    assert two["nodes"][2]["dependencies"] == ["node_softmax"] and two["nodes"][1]["dependencies"] == []
    assert [k for k, _, _ in runtime.plan(two)] == ["softmax", "nms", "topk"]      # the probabilities are an output: no fusion
