"""Writes the ONNX models of tests/cpp/test_onnx_import.cpp under tests/golden/onnx/, every model twice:
as protobuf text (.prototxt) and as binary protobuf (.onnx), from one description below.

The graphs restate those the nGraph tree's importer tests load (test/onnx/onnx_import_quant.in.cpp with
test/models/onnx/{quantize_linear*, dequant_lin, dequantize_linear_*, quant_conv_lin, qlinear_conv_2d,
qlinear_conv_3d, qlinear_matmul*, conv_integer*, matmul_integer*}.prototxt): same operators, shapes,
attributes, initializers and opset versions, so that the expected vectors of those tests apply.
Neither the `onnx` nor the `protobuf` package is used: the few messages are encoded by hand
(field numbers of onnx.proto), which also makes the files an independent check of the reader.

    python tests/golden/make_onnx_models.py
"""
import os
import struct

FLOAT, UINT8, INT8, INT32, INT64 = 1, 2, 3, 6, 7
HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "onnx")


# ---------------------------------------------------------------- a message = list of (field, kind, value)
# kinds: "int" (varint), "float" (fixed32), "bytes" (string / bytes), "msg" (nested list), "enum" (name, number)
FIELD_NUMBERS = {
    "model": {"ir_version": 1, "producer_name": 2, "graph": 7, "opset_import": 8},
    "opset": {"domain": 1, "version": 2},
    "graph": {"node": 1, "name": 2, "initializer": 5, "input": 11, "output": 12},
    "node": {"input": 1, "output": 2, "name": 3, "op_type": 4, "attribute": 5},
    "attribute": {"name": 1, "f": 2, "i": 3, "s": 4, "t": 5, "floats": 7, "ints": 8, "type": 20},
    "tensor": {"dims": 1, "data_type": 2, "float_data": 4, "int32_data": 5, "int64_data": 7, "name": 8, "raw_data": 9},
    "value_info": {"name": 1, "type": 2},
    "type": {"tensor_type": 1},
    "tensor_type": {"elem_type": 1, "shape": 2},
    "shape": {"dim": 1},
    "dim": {"dim_value": 1},
}
ATTRIBUTE_TYPES = {"FLOAT": 1, "INT": 2, "STRING": 3, "TENSOR": 4, "FLOATS": 6, "INTS": 7}


def varint(v):
    v &= (1 << 64) - 1  # negative int64 values take ten bytes
    out = bytearray()
    while True:
        b = v & 0x7F
        v >>= 7
        if v:
            out.append(b | 0x80)
        else:
            out.append(b)
            return bytes(out)


def encode(kind, fields):
    out = bytearray()
    for name, fkind, value in fields:
        number = FIELD_NUMBERS[kind][name]
        if fkind == "int":
            out += varint(number << 3 | 0) + varint(value)
        elif fkind == "enum":
            out += varint(number << 3 | 0) + varint(value[1])
        elif fkind == "float":
            out += varint(number << 3 | 5) + struct.pack("<f", value)
        elif fkind == "bytes":
            data = value if isinstance(value, bytes) else value.encode()
            out += varint(number << 3 | 2) + varint(len(data)) + data
        else:
            sub = encode(fkind[4:], value)
            out += varint(number << 3 | 2) + varint(len(sub)) + sub
    return bytes(out)


def quote(data):
    data = data if isinstance(data, bytes) else data.encode()
    out = []
    for b in data:
        c = chr(b)
        if c in '"\\':
            out.append("\\" + c)
        elif 32 <= b < 127:
            out.append(c)
        else:
            out.append("\\%03o" % b)
    return '"' + "".join(out) + '"'


def text(kind, fields, indent=0):
    pad = "  " * indent
    lines = []
    for name, fkind, value in fields:
        if fkind == "int":
            lines.append("%s%s: %d" % (pad, name, value))
        elif fkind == "enum":
            lines.append("%s%s: %s" % (pad, name, value[0]))
        elif fkind == "float":
            lines.append("%s%s: %s" % (pad, name, repr(struct.unpack("<f", struct.pack("<f", value))[0])))
        elif fkind == "bytes":
            lines.append("%s%s: %s" % (pad, name, quote(value)))
        else:
            lines.append("%s%s {" % (pad, name))
            lines.append(text(fkind[4:], value, indent + 1))
            lines.append("%s}" % pad)
    return "\n".join(l for l in lines if l != "")


# ---------------------------------------------------------------- ONNX pieces
def value_info(name, elem_type, shape):
    dims = [("dim", "msg:dim", [("dim_value", "int", d)]) for d in shape]
    return [("name", "bytes", name), ("type", "msg:type", [("tensor_type", "msg:tensor_type", [("elem_type", "int", elem_type), ("shape", "msg:shape", dims)])])]


def tensor(name, data_type, shape, values=None, raw=None):
    fields = [("dims", "int", d) for d in shape] + [("data_type", "int", data_type)]
    if raw is not None:
        fields.append(("raw_data", "bytes", raw))
    elif data_type == FLOAT:
        fields += [("float_data", "float", v) for v in values]
    elif data_type == INT64:
        fields += [("int64_data", "int", v) for v in values]
    else:
        fields += [("int32_data", "int", v) for v in values]
    return fields + [("name", "bytes", name)]


def attribute(name, value):
    if value is None:  # filled in by patch_constant_nodes
        return [("name", "bytes", name)]
    if isinstance(value, int):
        return [("name", "bytes", name), ("i", "int", value), ("type", "enum", ("INT", ATTRIBUTE_TYPES["INT"]))]
    if isinstance(value, str):
        return [("name", "bytes", name), ("s", "bytes", value), ("type", "enum", ("STRING", ATTRIBUTE_TYPES["STRING"]))]
    return [("name", "bytes", name)] + [("ints", "int", v) for v in value] + [("type", "enum", ("INTS", ATTRIBUTE_TYPES["INTS"]))]


def node(op_type, inputs, outputs, name="", **attributes):
    fields = [("input", "bytes", i) for i in inputs] + [("output", "bytes", o) for o in outputs]
    if name:
        fields.append(("name", "bytes", name))
    fields.append(("op_type", "bytes", op_type))
    fields += [("attribute", "msg:attribute", attribute(k, v)) for k, v in attributes.items()]
    return fields


def model(nodes, inputs, outputs, initializers=(), opset=10, ir_version=3, opset_domain=None):
    graph = [("node", "msg:node", n) for n in nodes] + [("name", "bytes", "test_graph")]
    graph += [("initializer", "msg:tensor", t) for t in initializers]
    graph += [("input", "msg:value_info", value_info(*i)) for i in inputs]
    graph += [("output", "msg:value_info", value_info(*o)) for o in outputs]
    opset_fields = ([("domain", "bytes", opset_domain)] if opset_domain is not None else []) + [("version", "int", opset)]
    return [("ir_version", "int", ir_version), ("producer_name", "bytes", "hipq tests"), ("graph", "msg:graph", graph), ("opset_import", "msg:opset", opset_fields)]


def quantize_linear(x_shape, scale_shape, zp_type=UINT8, zp_initializer=None, **attrs):
    inits = [tensor("y_zero_point", zp_type, scale_shape, raw=zp_initializer)] if zp_initializer is not None else []
    return model([node("QuantizeLinear", ["x", "y_scale", "y_zero_point"], ["y"], "node1", **attrs)],
                 [("x", FLOAT, x_shape), ("y_scale", FLOAT, scale_shape), ("y_zero_point", zp_type, scale_shape)], [("y", zp_type, x_shape)], inits)


def dequantize_linear(x_type, x_shape, scale_shape, initializers=(), opset=10, **attrs):
    return model([node("DequantizeLinear", ["x", "x_scale", "x_zero_point"], ["y"], "node1", **attrs)],
                 [("x", x_type, x_shape), ("x_scale", FLOAT, scale_shape), ("x_zero_point", x_type, scale_shape)], [("y", FLOAT, x_shape)], initializers, opset)


def qlinear_conv(x_shape, w_shape, y_shape, w_type=UINT8, y_type=UINT8, initializers=(), opset=10, bias=False, **attrs):
    names = ["x", "x_scale", "x_zero_point", "w", "w_scale", "w_zero_point", "y_scale", "y_zero_point"] + (["bias"] if bias else [])
    inputs = [("x", UINT8, x_shape), ("x_scale", FLOAT, []), ("x_zero_point", UINT8, []), ("w", w_type, w_shape), ("w_scale", FLOAT, []), ("w_zero_point", w_type, []),
              ("y_scale", FLOAT, []), ("y_zero_point", y_type, [])]
    return model([node("QLinearConv", names, ["y"], "node1", **attrs)], inputs, [("y", y_type, y_shape)], initializers, opset)


def qlinear_matmul(a_shape, b_shape, y_shape):
    names = ["T1", "a_scale", "a_zero_point", "T2", "b_scale", "b_zero_point", "y_scale", "y_zero_point"]
    inputs = [("T1", UINT8, a_shape), ("a_scale", FLOAT, []), ("a_zero_point", UINT8, []), ("T2", UINT8, b_shape), ("b_scale", FLOAT, []), ("b_zero_point", UINT8, []),
              ("y_scale", FLOAT, []), ("y_zero_point", UINT8, [])]
    return model([node("QLinearMatMul", names, ["T3"], "node1")], inputs, [("T3", UINT8, y_shape)], ir_version=4)


def conv_integer(y_shape, zero_point=True, **attrs):
    names = ["x", "w"] + (["x_zero_point"] if zero_point else [])
    inputs = [("x", UINT8, [1, 1, 3, 3]), ("w", UINT8, [1, 1, 2, 2])] + ([("x_zero_point", UINT8, [])] if zero_point else [])
    return model([node("ConvInteger", names, ["y"], "node1", group=1, auto_pad="NOTSET", **attrs)], inputs, [("y", INT32, y_shape)], ir_version=5, opset_domain="")


def matmul_integer(a_shape, b_shape, y_shape, zero_points=True):
    names = ["a", "b"] + (["a_zero_point", "b_zero_point"] if zero_points else [])
    inputs = [("a", UINT8, a_shape), ("b", UINT8, b_shape)] + ([("a_zero_point", UINT8, []), ("b_zero_point", UINT8, [])] if zero_points else [])
    return model([node("MatMulInteger", names, ["y"], "node1")], inputs, [("y", INT32, y_shape)], ir_version=5, opset_domain="")


def scalars_for_conv_lin():
    return [tensor("x_zero_point", UINT8, [], raw=b"\x00"), tensor("x_scale", FLOAT, [], [1.0]), tensor("w_zero_point", INT8, [], raw=b"\x00"), tensor("w_scale", FLOAT, [], [1.0]),
            tensor("y_zero_point", INT8, [], raw=b"\x00"), tensor("y_scale", FLOAT, [], [16.0]), tensor("w", INT8, [1, 1, 3, 3], [1, 0, 2, 1, 0, 2, 1, 0, 2])]


MODELS = {
    # QuantizeLinear: zero point from an initializer; as inputs; per-axis scales (axis 0, axis -2)
    "quantize_linear": quantize_linear([2, 2], [], zp_initializer=b"\x00"),
    "quantize_linear_zero_point": quantize_linear([6], []),
    "quantize_linear_axis_zero": quantize_linear([3, 4], [3], axis=0),
    "quantize_linear_axis_negative": quantize_linear([3, 4], [3], axis=-2),
    # DequantizeLinear: constants from initializers (opset 4 file); u8 / i8 scalars; per-axis forms
    "dequantize_linear_initializers": dequantize_linear(UINT8, [2, 2], [], [tensor("x_zero_point", UINT8, [], raw=b"\x00"), tensor("x_scale", FLOAT, [], [4.0])], opset=4),
    "dequantize_linear_u8": dequantize_linear(UINT8, [4], []),
    "dequantize_linear_i8": dequantize_linear(INT8, [4], []),
    "dequantize_linear_axis0_u8": dequantize_linear(UINT8, [3, 4], [3], axis=0),
    "dequantize_linear_axis1_i8": dequantize_linear(INT8, [3, 4], [4], axis=1),
    "dequantize_linear_axis1_4d": dequantize_linear(UINT8, [2, 3, 2, 4], [3], axis=1),
    "dequantize_linear_axis_negative": dequantize_linear(UINT8, [3, 4], [3], axis=-2),
    # QLinearConv: everything but the data from initializers, i8 filter declared u8 in the input list (the initializer counts)
    "qlinear_conv_initializers": qlinear_conv([1, 1, 9, 9], [1, 1, 3, 3], [1, 1, 9, 9], w_type=UINT8, y_type=INT8, initializers=scalars_for_conv_lin(), opset=8, pads=[1, 1, 1, 1]),
    "qlinear_conv_2d": qlinear_conv([1, 1, 7, 7], [1, 1, 1, 1], [1, 1, 7, 7], group=1, auto_pad="NOTSET"),
    "qlinear_conv_3d": qlinear_conv([1, 1, 4, 4, 4], [1, 1, 1, 1, 1], [1, 1, 4, 4, 4], group=1, auto_pad="NOTSET", pads=[2, 2, 2, 2, 2, 2], strides=[2, 2, 2]),
    "qlinear_matmul": qlinear_matmul([2, 4], [4, 3], [2, 3]),
    "qlinear_matmul_3d": qlinear_matmul([2, 2, 4], [2, 4, 3], [2, 2, 3]),
    "conv_integer": conv_integer([1, 1, 2, 2]),
    "conv_integer_no_zero_point": conv_integer([1, 1, 2, 2], zero_point=False),
    "conv_integer_pads": conv_integer([1, 1, 4, 4], pads=[1, 1, 1, 1]),
    "matmul_integer": matmul_integer([4, 3], [3, 2], [4, 2]),
    "matmul_integer_no_zero_point": matmul_integer([4, 3], [3, 2], [4, 2], zero_points=False),
    "matmul_integer_scalar": matmul_integer([1, 1], [1, 1], [1, 1]),
    "matmul_integer_4d": matmul_integer([1, 2, 3, 4], [1, 2, 4, 3], [1, 2, 3, 3]),
    "matmul_integer_4d_no_zero_point": matmul_integer([1, 2, 3, 4], [1, 2, 4, 3], [1, 2, 3, 3], zero_points=False),
    # stack axes broadcast numpy-style: a stack of one matrix against two, two stack axes against each other, a matrix against a stack; stacks that do not fit
    "matmul_integer_broadcast_3d": matmul_integer([2, 3, 4], [1, 4, 3], [2, 3, 3]),
    "matmul_integer_broadcast_4d": matmul_integer([2, 1, 3, 4], [1, 3, 4, 2], [2, 3, 3, 2]),
    "matmul_integer_matrix_by_stack": matmul_integer([3, 4], [2, 4, 3], [2, 3, 3]),
    "matmul_integer_stacks_clash": matmul_integer([2, 3, 4], [3, 4, 3], [2, 3, 3]),
    # QLinearConv in two groups: a 1 x 1 filter a channel (unit scales, zero zero points)
    "qlinear_conv_groups": qlinear_conv(
        [1, 2, 2, 2], [2, 1, 1, 1], [1, 2, 2, 2], w_type=INT8, y_type=INT8,
        initializers=[tensor("x_scale", FLOAT, [], [1.0]), tensor("x_zero_point", UINT8, [], raw=b"\x00"), tensor("w", INT8, [2, 1, 1, 1], [2, 3]), tensor("w_scale", FLOAT, [], [1.0]),
                      tensor("w_zero_point", INT8, [], raw=b"\x00"), tensor("y_scale", FLOAT, [], [1.0]), tensor("y_zero_point", INT8, [], raw=b"\x00")],
        group=2),
    # automatic padding: a 3 x 3 window over 4 x 4 at stride 2 needs one more row and column, below the data (SAME_LOWER) or above it (SAME_UPPER)
    "conv_integer_same_upper": model([node("ConvInteger", ["x", "w"], ["y"], "node1", auto_pad="SAME_UPPER", strides=[2, 2])], [("x", UINT8, [1, 1, 4, 4]), ("w", UINT8, [1, 1, 3, 3])],
                                     [("y", INT32, [1, 1, 2, 2])]),
    "conv_integer_same_lower": model([node("ConvInteger", ["x", "w"], ["y"], "node1", auto_pad="SAME_LOWER", strides=[2, 2])], [("x", UINT8, [1, 1, 4, 4]), ("w", UINT8, [1, 1, 3, 3])],
                                     [("y", INT32, [1, 1, 2, 2])]),
    # a chain with glue: DequantizeLinear -> Relu -> QuantizeLinear with constants from Constant nodes
    "dequantize_relu_quantize": model(
        [
            node("Constant", [], ["scale"], "c_scale", value=None),
            node("Constant", [], ["zero"], "c_zero", value=None),
            node("DequantizeLinear", ["x", "scale", "zero"], ["real"], "dq"),
            node("Relu", ["real"], ["positive"], "relu"),
            node("QuantizeLinear", ["positive", "scale", "zero"], ["y"], "q"),
        ],
        [("x", INT8, [2, 3])],
        [("y", INT8, [2, 3])],
    ),
    # QLinearConv with the optional ninth input: an int32 bias (requantization scale 0.5 * 0.25 / 0.125 = 1)
    "qlinear_conv_bias": qlinear_conv(
        [1, 1, 2, 2], [1, 1, 1, 1], [1, 1, 2, 2], w_type=INT8, y_type=INT8,
        initializers=[tensor("x_scale", FLOAT, [], [0.5]), tensor("x_zero_point", UINT8, [], raw=b"\x00"), tensor("w", INT8, [1, 1, 1, 1], [2]), tensor("w_scale", FLOAT, [], [0.25]),
                      tensor("w_zero_point", INT8, [], raw=b"\x00"), tensor("y_scale", FLOAT, [], [0.125]), tensor("y_zero_point", INT8, [], raw=b"\x00"), tensor("bias", INT32, [1], [10])],
        bias=True),
    "unsupported_operator": model([node("Softplus", ["x"], ["y"], "node1")], [("x", FLOAT, [2])], [("y", FLOAT, [2])]),
}


def patch_constant_nodes(fields):
    """Constant nodes carry their tensor in a `value` attribute of kind TENSOR"""
    graph = [f for f in fields if f[0] == "graph"][0][2]
    tensors = {"c_scale": tensor("", FLOAT, [], [0.5]), "c_zero": tensor("", INT8, [], raw=b"\x00")}
    for i, (name, kind, value) in enumerate(graph):
        if name != "node":
            continue
        node_name = [f[2] for f in value if f[0] == "name"]
        if node_name and node_name[0] in tensors:
            value[:] = [f for f in value if f[0] != "attribute"]
            value.append(("attribute", "msg:attribute", [("name", "bytes", "value"), ("t", "msg:tensor", tensors[node_name[0]]), ("type", "enum", ("TENSOR", ATTRIBUTE_TYPES["TENSOR"]))]))


def main():
    os.makedirs(OUT, exist_ok=True)
    for name, fields in MODELS.items():
        patch_constant_nodes(fields)
        with open(os.path.join(OUT, name + ".prototxt"), "w") as f:
            f.write(text("model", fields) + "\n")
        with open(os.path.join(OUT, name + ".onnx"), "wb") as f:
            f.write(encode("model", fields))
    print("wrote", 2 * len(MODELS), "files to", OUT)


if __name__ == "__main__":
    main()
