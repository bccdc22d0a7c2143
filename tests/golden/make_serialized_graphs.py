"""Writes tests/golden/serialized/*.json: quantized graphs in the JSON layout nGraph's serializer
produces, restated here from its source (src/ngraph/serializer.cpp:556-581 function, :2661-2724 node
header, :2852-2869 Constant, :3339-3346 Parameter, :3399-3453 Quantize / QuantizedConvolution /
QuantizedDot, :2997-3003 Dequantize, :3474-3479 Result, :3681-3694 attribute-visitor ops) independently
of this repository's C++ writer, so that the reader is checked against the format and not against
itself.  nGraph holds no serialized quantized model of its own (its fused quantized ops have no JSON
form), so the graphs are the ones its backend tests build in C++:

  qconv_i32_output.json   test/backend/quantized_convolution.in.cpp  quantized_conv_int32_output
  qdot_u8u8.json          test/backend/quantized_dot.in.cpp:31-76     quantized_dot_u8u8
  qdot_i32_output.json    test/backend/quantized_dot.in.cpp:78-115    quantized_dot_int32_output
  quantize_dequantize.json test/backend/quantize_dequantize.in.cpp:31-108  quantize, then dequantize
  legacy_scale_subgraph.json  float glue in the layout of nGraph's oldest files (no op_version, no
                          Result nodes, element types as objects; cf. test/models/mxnet/Graph_fprop_sigmoid.json)
  qconv_3x3_64ch_b128.json  the 3x3 / 64-channel / 56x56 layer at batch 128 with a constant filter

Run from the repository root:  python tests/golden/make_serialized_graphs.py
"""
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "serialized")

C_TYPE = {"f32": "float", "u8": "uint8_t", "i8": "int8_t", "i32": "int32_t"}


class Graph:
    """node names carry a running instance number, as Node::get_name() gives them"""

    def __init__(self, name, legacy=False):
        self.name, self.ops, self.count, self.legacy = name, [], 0, legacy

    def node(self, op, inputs=(), version=0, **attrs):
        name = "%s_%d" % (op, self.count)
        self.count += 1
        n = {"name": name, "op": op, "outputs": [name + "_0"]}
        if not self.legacy:
            n["op_version"] = version
        if inputs or self.legacy:
            n["inputs"] = list(inputs)
        n.update(attrs)
        self.ops.append(n)
        return name

    def etype(self, t):
        if not self.legacy:
            return C_TYPE[t]
        return {"bitwidth": 32, "c_type_string": C_TYPE[t], "is_quantized": False, "is_real": t == "f32", "is_signed": t != "u8"}

    def parameter(self, t, shape):
        extra = {} if self.legacy else {"cacheable": False}
        return self.node("Parameter", element_type=self.etype(t), shape=list(shape), **extra)

    def constant(self, t, shape, values):
        return self.node("Constant", element_type=self.etype(t), shape=list(shape), value=[str(v) for v in values])

    def result(self, arg):
        return self.node("Result", [arg], needs_default_layout=False)

    def function(self, parameters, results):
        return [{"name": self.name, "ops": self.ops, "parameters": parameters, "result": results}]


def write(fname, js, indent):
    text = json.dumps(js, sort_keys=True, indent=indent or None, separators=(",", ": ") if indent else (",", ":"))
    with open(os.path.join(OUT, fname), "w") as f:
        f.write(text)
    print(fname, len(text), "bytes")


def qconv_attrs(out_t):
    return dict(
        window_movement_strides=[1, 1],
        window_dilation_strides=[1, 1],
        padding_below=[1, 1],
        padding_above=[1, 1],
        data_dilation_strides=[1, 1],
        output_type=C_TYPE[out_t],
        input_axes=[],
        filter_axes=[],
        output_axes=[],
    )


def qconv_i32_output():
    g = Graph("Function_0")
    A = g.parameter("u8", (1, 1, 3, 4))
    B = g.parameter("u8", (1, 1, 3, 3))
    C = g.parameter("f32", ())
    D = g.constant("u8", (), [0])
    E = g.parameter("f32", ())
    F = g.constant("u8", (), [0])
    G = g.parameter("f32", ())
    H = g.constant("i32", (), [0])
    cv = g.node("QuantizedConvolution", [A, B, C, D, E, F, G, H], **qconv_attrs("i32"))
    r = g.result(cv)
    write("qconv_i32_output.json", g.function([A, B, C, E, G], [r]), 4)


def qdot(fname, b_t, out_t, scales):
    g = Graph("Function_1")
    A = g.parameter("u8", (1, 2))
    B = g.parameter(b_t, (2, 3))
    s0 = g.constant("f32", (), [scales[0]])
    z0 = g.constant("u8", (), [0])
    s1 = g.constant("f32", (), [scales[1]])
    z1 = g.constant(b_t, (), [0])
    s2 = g.constant("f32", (), [scales[2]])
    z2 = g.constant(out_t, (), [0])
    qd = g.node(
        "QuantizedDot",
        [A, B, s0, z0, s1, z1, s2, z2],
        reduction_axes_count=1,
        output_type=C_TYPE[out_t],
        input0_axes=[],
        input1_axes=[],
        output_axes=[],
    )
    r = g.result(qd)
    write(fname, g.function([A, B], [r]), 0)


def quantize_dequantize():
    g = Graph("Function_2")
    X = g.parameter("f32", (4, 3))
    scale = g.constant("f32", (), [2])
    offset = g.constant("u8", (), [1])
    q = g.node("Quantize", [X, scale, offset], type="uint8_t", axes=[], round_mode=4)  # ROUND_NEAREST_TOWARD_EVEN
    dq = g.node("Dequantize", [q, scale, offset], type="float", axes=[])
    r0, r1 = g.result(q), g.result(dq)
    write("quantize_dequantize.json", g.function([X], [r0, r1]), 2)


def legacy_scale_subgraph():
    g = Graph("Function_3", legacy=True)
    a = g.parameter("f32", (2, 3))
    b = g.parameter("f32", (2, 3))
    ab = g.node("Abs", [a])
    m = g.node("Maximum", [ab, b])
    two = g.constant("f32", (), [2])
    bc = g.node("Broadcast", [two], shape=[2, 3], axes=[0, 1])
    d = g.node("Divide", [m, bc])
    s = g.node("Add", [d, a])
    p = g.node("Multiply", [s, b])
    write("legacy_scale_subgraph.json", g.function([a, b], [p]), 0)


def qconv_3x3_64ch_b128():
    rng = np.random.default_rng(20240607)
    filt = rng.integers(-127, 128, 64 * 64 * 3 * 3)
    g = Graph("Function_4")
    data = g.parameter("u8", (128, 64, 56, 56))
    w = g.constant("i8", (64, 64, 3, 3), filt.tolist())
    s0, z0 = g.constant("f32", (), ["0.0199999996"]), g.constant("u8", (), [0])
    s1, z1 = g.constant("f32", (), ["0.00499999989"]), g.constant("i8", (), [0])
    s2, z2 = g.constant("f32", (), ["0.100000001"]), g.constant("i8", (), [0])
    cv = g.node("QuantizedConvolution", [data, w, s0, z0, s1, z1, s2, z2], **qconv_attrs("i8"))
    r = g.result(cv)
    write("qconv_3x3_64ch_b128.json", g.function([data], [r]), 0)


if __name__ == "__main__":
    os.makedirs(OUT, exist_ok=True)
    qconv_i32_output()
    qdot("qdot_u8u8.json", "u8", "u8", [2, 1, 2])
    qdot("qdot_i32_output.json", "i8", "i32", [1, 1, 1])
    quantize_dequantize()
    legacy_scale_subgraph()
    qconv_3x3_64ch_b128()
