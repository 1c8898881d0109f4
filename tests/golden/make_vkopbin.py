#!/usr/bin/env python3
"""Writes the .vkopbin fixtures next to this file (run from anywhere):

  classifier_head.vkopbin   logits [8,1000] -> Softmax(axis -1) -> TopK(K 5): values, indices.
                            The softmax output has one reader and is no model output: fusable.
  classifier_head_k_input.vkopbin
                            the same head as ONNX stores it: K is the TopK's second input, an int64
                            initializer; the probabilities are a model output too: not fusable.
  detection_tail.vkopbin    scores [2,3,300] and boxes [2,300,4] -> Nms: records.
                            Attributes of all five tagged kinds appear (a string and two lists ride
                            along, unused by the operator).

  detection_chain.vkopbin   class scores [2,80,840] -> Softmax(axis 1) -> Reduce(max, axes [1], keepdims 0) ->
                            TopK(K 30): the detection-style post-processing (example/yolo/main.cpp:60-127).

  two_heads.vkopbin         a classifier head (probabilities and top-7, the probabilities an output too) beside a
                            detection tail in one model: two nodes in the first level, a dependency into the second.

add_conv_model.vkopbin is not written here: it is the reference's own model file
(model/add_conv_model.vkopbin, made by its converter), kept as a reading fixture.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from vkop_amd import vkopbin  # noqa: E402


def shape(name, dims):
    return {"name": name, "shape": list(dims)}


def main():
    head = vkopbin.write_model(
        [shape("logits", (8, 1000))], [shape("values", (8, 5)), shape("indices", (8, 5))],
        [{"op_type": "Softmax", "name": "node_softmax", "attributes": {"axis": -1},
          "inputs": [shape("logits", (8, 1000))], "outputs": [shape("probs", (8, 1000))]},
         {"op_type": "TopK", "name": "node_topk", "attributes": {"K": 5, "axis": -1, "largest": 1, "sorted": 1},
          "inputs": [shape("probs", (8, 1000))], "outputs": [shape("values", (8, 5)), shape("indices", (8, 5))]}])
    open(os.path.join(HERE, "classifier_head.vkopbin"), "wb").write(head)

    head_k = vkopbin.write_model(
        [shape("logits", (4, 1000))], [shape("probs", (4, 1000)), shape("values", (4, 7)), shape("indices", (4, 7))],
        [{"op_type": "Softmax", "name": "node_softmax", "attributes": {"axis": 1},
          "inputs": [shape("logits", (4, 1000))], "outputs": [shape("probs", (4, 1000))]},
         {"op_type": "TopK", "name": "node_topk", "attributes": {"axis": -1},
          "inputs": [shape("probs", (4, 1000)), shape("k_value", (1,))],
          "outputs": [shape("values", (4, 7)), shape("indices", (4, 7))]}],
        {"k_value": np.array([7], dtype=np.int64)})
    open(os.path.join(HERE, "classifier_head_k_input.vkopbin"), "wb").write(head_k)

    tail = vkopbin.write_model(
        [shape("boxes", (2, 300, 4)), shape("scores", (2, 3, 300))], [shape("selected", (1800, 3))],
        [{"op_type": "Nms", "name": "node_nms",
          "attributes": {"center_point_box": 0, "iou_threshold": 0.5, "score_threshold": 0.25,
                         "max_output_boxes_per_class": 0, "note": "detection tail", "strides": [8, 16, 32],
                         "anchors": [1.5, 2.25]},
          "inputs": [shape("boxes", (2, 300, 4)), shape("scores", (2, 3, 300))], "outputs": [shape("selected", (1800, 3))]}])
    open(os.path.join(HERE, "detection_tail.vkopbin"), "wb").write(tail)

    chain = vkopbin.write_model(
        [shape("scores", (2, 80, 840))], [shape("values", (2, 30)), shape("anchors", (2, 30))],
        [{"op_type": "Softmax", "name": "node_softmax", "attributes": {"axis": 1},
          "inputs": [shape("scores", (2, 80, 840))], "outputs": [shape("probs", (2, 80, 840))]},
         {"op_type": "Reduce", "name": "node_max", "attributes": {"reduce_op": "max", "axes": [1], "keepdims": 0},
          "inputs": [shape("probs", (2, 80, 840))], "outputs": [shape("best", (2, 840))]},
         {"op_type": "TopK", "name": "node_topk", "attributes": {"K": 30, "axis": -1},
          "inputs": [shape("best", (2, 840))], "outputs": [shape("values", (2, 30)), shape("anchors", (2, 30))]}])
    open(os.path.join(HERE, "detection_chain.vkopbin"), "wb").write(chain)

    two = vkopbin.write_model(
        [shape("logits", (4, 1000)), shape("boxes", (1, 200, 4)), shape("scores", (1, 4, 200))],
        [shape("probs", (4, 1000)), shape("values", (4, 7)), shape("indices", (4, 7)), shape("selected", (800, 3))],
        [{"op_type": "Softmax", "name": "node_softmax", "attributes": {"axis": -1},
          "inputs": [shape("logits", (4, 1000))], "outputs": [shape("probs", (4, 1000))]},
         {"op_type": "Nms", "name": "node_nms", "attributes": {"iou_threshold": 0.4, "score_threshold": 0.5},
          "inputs": [shape("boxes", (1, 200, 4)), shape("scores", (1, 4, 200))], "outputs": [shape("selected", (800, 3))]},
         {"op_type": "TopK", "name": "node_topk", "attributes": {"K": 7},
          "inputs": [shape("probs", (4, 1000))], "outputs": [shape("values", (4, 7)), shape("indices", (4, 7))]}])
    open(os.path.join(HERE, "two_heads.vkopbin"), "wb").write(two)


if __name__ == "__main__":
    main()
