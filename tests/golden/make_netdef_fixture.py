#!/usr/bin/env python3
"""Writes tests/golden/netdef_unpacked.pb and netdef_packed.pb: one NetDef serialized by the
google.protobuf package (an independent implementation of the wire format), for the reader in
include/mace_hip_net.h to parse (tests/cpp/test_net.cc, mode `fixture`).

The message descriptors are built here from the schema the reader follows (the reference's
mace/proto/mace.proto:24-117: message names, field names, numbers and types), so neither protoc
nor generated code is needed.  The same NetDef is written twice: with the repeated scalar fields
declared as in the schema (proto2: unpacked unless marked packed) and with every one of them
marked packed -- a conforming reader accepts either form for any repeated scalar.  The values
include what a hand-written reader gets wrong first: negative int32 / int64 (ten-byte varints),
floats in both repeated forms, empty strings, fields the reader does not know (device_type,
mem_id, float_data, node_id ...) and nested messages in sequence.

    python tests/golden/make_netdef_fixture.py
"""
import os

from google.protobuf import descriptor_pb2, descriptor_pool, message_factory

F = descriptor_pb2.FieldDescriptorProto
OPT, REP = F.LABEL_OPTIONAL, F.LABEL_REPEATED
HERE = os.path.dirname(os.path.abspath(__file__))

# (name, number, label, type, type_name or None, packed-in-schema)
SCHEMA = {
    "ConstTensor": [("dims", 1, REP, F.TYPE_INT64, None, False), ("data_type", 2, OPT, F.TYPE_ENUM, ".mace.DataType", False),
                    ("float_data", 3, REP, F.TYPE_FLOAT, None, True), ("int32_data", 4, REP, F.TYPE_INT32, None, True),
                    ("name", 5, OPT, F.TYPE_STRING, None, False), ("offset", 6, OPT, F.TYPE_INT64, None, False),
                    ("data_size", 7, OPT, F.TYPE_INT64, None, False), ("scale", 8, OPT, F.TYPE_FLOAT, None, False),
                    ("zero_point", 9, OPT, F.TYPE_INT32, None, False), ("minval", 10, OPT, F.TYPE_FLOAT, None, False),
                    ("maxval", 11, OPT, F.TYPE_FLOAT, None, False), ("quantized", 12, OPT, F.TYPE_BOOL, None, False),
                    ("node_id", 100, OPT, F.TYPE_UINT32, None, False)],
    "Argument": [("name", 1, OPT, F.TYPE_STRING, None, False), ("f", 2, OPT, F.TYPE_FLOAT, None, False),
                 ("i", 3, OPT, F.TYPE_INT64, None, False), ("s", 4, OPT, F.TYPE_BYTES, None, False),
                 ("floats", 5, REP, F.TYPE_FLOAT, None, False), ("ints", 6, REP, F.TYPE_INT64, None, False)],
    "NodeInput": [("node_id", 1, OPT, F.TYPE_INT32, None, False), ("output_port", 2, OPT, F.TYPE_INT32, None, False)],
    "OutputShape": [("dims", 1, REP, F.TYPE_INT64, None, False)],
    "QuantizeActivationInfo": [("scale", 1, OPT, F.TYPE_FLOAT, None, False), ("zero_point", 2, OPT, F.TYPE_INT32, None, False),
                               ("minval", 3, OPT, F.TYPE_FLOAT, None, False), ("maxval", 4, OPT, F.TYPE_FLOAT, None, False)],
    "OperatorDef": [("input", 1, REP, F.TYPE_STRING, None, False), ("output", 2, REP, F.TYPE_STRING, None, False),
                    ("name", 3, OPT, F.TYPE_STRING, None, False), ("type", 4, OPT, F.TYPE_STRING, None, False),
                    ("device_type", 5, OPT, F.TYPE_INT32, None, False), ("arg", 6, REP, F.TYPE_MESSAGE, ".mace.Argument", False),
                    ("output_shape", 7, REP, F.TYPE_MESSAGE, ".mace.OutputShape", False),
                    ("output_type", 8, REP, F.TYPE_ENUM, ".mace.DataType", False),
                    ("quantize_info", 9, REP, F.TYPE_MESSAGE, ".mace.QuantizeActivationInfo", False),
                    ("mem_id", 10, REP, F.TYPE_INT32, None, False), ("node_id", 100, OPT, F.TYPE_UINT32, None, False),
                    ("op_id", 101, OPT, F.TYPE_UINT32, None, False), ("padding", 102, OPT, F.TYPE_UINT32, None, False),
                    ("node_input", 103, REP, F.TYPE_MESSAGE, ".mace.NodeInput", False),
                    ("out_max_byte_size", 104, REP, F.TYPE_INT32, None, False)],
    "InputOutputInfo": [("name", 1, OPT, F.TYPE_STRING, None, False), ("node_id", 2, OPT, F.TYPE_INT32, None, False),
                        ("dims", 3, REP, F.TYPE_INT32, None, False), ("max_byte_size", 4, OPT, F.TYPE_INT32, None, False),
                        ("data_type", 5, OPT, F.TYPE_ENUM, ".mace.DataType", False),
                        ("data_format", 6, OPT, F.TYPE_INT32, None, False), ("scale", 7, OPT, F.TYPE_FLOAT, None, False),
                        ("zero_point", 8, OPT, F.TYPE_INT32, None, False), ("alias", 100, OPT, F.TYPE_STRING, None, False)],
    "NetDef": [("op", 1, REP, F.TYPE_MESSAGE, ".mace.OperatorDef", False), ("arg", 2, REP, F.TYPE_MESSAGE, ".mace.Argument", False),
               ("tensors", 3, REP, F.TYPE_MESSAGE, ".mace.ConstTensor", False),
               ("data_type", 4, OPT, F.TYPE_ENUM, ".mace.DataType", False), ("name", 5, OPT, F.TYPE_STRING, None, False),
               ("data_offset", 6, OPT, F.TYPE_INT32, None, False), ("data_size", 7, OPT, F.TYPE_INT32, None, False),
               ("infer_order", 8, OPT, F.TYPE_INT32, None, False),
               ("input_info", 100, REP, F.TYPE_MESSAGE, ".mace.InputOutputInfo", False),
               ("output_info", 101, REP, F.TYPE_MESSAGE, ".mace.InputOutputInfo", False)],
}
DATA_TYPES = ["DT_INVALID", "DT_FLOAT", "DT_UINT8", "DT_HALF", "DT_INT32", "DT_FLOAT16", "DT_BFLOAT16", "DT_INT16",
              "DT_INT8", "DT_UINT16", "DT_UINT32", "DT_BOOL"]


def messages(all_packed, package):
    fd = descriptor_pb2.FileDescriptorProto(name="%s.proto" % package, package=package, syntax="proto2")
    en = fd.enum_type.add(name="DataType")
    for i, n in enumerate(DATA_TYPES):
        en.value.add(name=n, number=i)
    for msg, fields in SCHEMA.items():
        m = fd.message_type.add(name=msg)
        for (name, number, label, ftype, type_name, packed) in fields:
            f = m.field.add(name=name, number=number, label=label, type=ftype)
            if type_name:
                f.type_name = type_name.replace(".mace.", ".%s." % package)
            scalar = ftype not in (F.TYPE_MESSAGE, F.TYPE_STRING, F.TYPE_BYTES)
            if label == REP and scalar and (packed or all_packed):
                f.options.packed = True
    pool = descriptor_pool.DescriptorPool()
    pool.Add(fd)
    return {n: message_factory.GetMessageClass(pool.FindMessageTypeByName("%s.%s" % (package, n))) for n in SCHEMA}


def build(M):
    net = M["NetDef"](name="fixture_net", data_type=1, data_offset=0, data_size=4096, infer_order=1)
    ga = net.arg.add(name="net_level_arg", i=7)                  # a NetDef field the reader skips
    del ga
    op = net.op.add(name="conv_a", type="Conv2D", device_type=0, node_id=11, op_id=5, padding=3)
    op.input.extend(["in_q", "conv_a/filter", "conv_a/bias"])
    op.output.append("act_a")
    op.arg.add(name="T", i=2)
    op.arg.add(name="strides", ints=[2, 1])
    op.arg.add(name="padding_values", ints=[-1, 0, 70000000000])  # negative and > 32 bits
    op.arg.add(name="max_limit", f=6.0)
    op.arg.add(name="activation", s=b"RELUX")
    op.arg.add(name="coeffs", floats=[0.25, -1.5, 3.0e-5])
    op.arg.add(name="neg", i=-123456789012)
    op.arg.add(name="", s=b"")                                    # empty name, empty bytes
    op.output_shape.add(dims=[64, 56, 56, 128])
    op.output_type.append(2)
    q = op.quantize_info.add(scale=0.023529412, zero_point=-7, minval=-0.5, maxval=6.0)
    del q
    op.mem_id.extend([3, -1])
    op.node_input.add(node_id=9, output_port=1)
    op.out_max_byte_size.extend([1024, 2048])
    op2 = net.op.add(name="two_outputs", type="Split")
    op2.input.append("act_a")
    op2.output.extend(["s0", "s1"])
    op2.output_shape.add(dims=[64, 56, 56, 64])
    op2.output_shape.add(dims=[])
    op2.output_type.extend([2, 4])
    op2.quantize_info.add(scale=0.5, zero_point=255)
    op2.quantize_info.add(scale=1.0e-3, zero_point=-2147483648)
    t = net.tensors.add(name="conv_a/filter", data_type=2, offset=256, data_size=128 * 128, scale=0.0123, zero_point=131,
                        minval=-1.6, maxval=1.5, quantized=True, node_id=4)
    t.dims.extend([128, 1, 1, 128])
    t2 = net.tensors.add(name="conv_a/bias", data_type=4, offset=256 + 128 * 128, data_size=128, scale=2.5e-4, zero_point=-3)
    t2.dims.append(128)
    t2.int32_data.extend([1, -2, 3])                              # inline data: skipped by the reader
    t3 = net.tensors.add(name="inline_floats", data_type=1, offset=0, data_size=2)
    t3.dims.extend([2])
    t3.float_data.extend([1.0, 2.0])
    i0 = net.input_info.add(name="in", node_id=1, max_byte_size=99, data_type=1, data_format=1, scale=0.0, zero_point=0,
                            alias="image")
    i0.dims.extend([64, 112, 112, 3])
    o0 = net.output_info.add(name="s1", data_type=4, scale=7.5, zero_point=-9)
    o0.dims.extend([64, 10])
    return net


def main():
    for tag, all_packed in (("unpacked", False), ("packed", True)):
        M = messages(all_packed, "mace" if not all_packed else "macep")
        data = build(M).SerializeToString(deterministic=True)
        with open(os.path.join(HERE, "netdef_%s.pb" % tag), "wb") as f:
            f.write(data)
        print("netdef_%s.pb: %d bytes" % (tag, len(data)))


if __name__ == "__main__":
    main()
