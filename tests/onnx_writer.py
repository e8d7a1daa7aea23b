"""A minimal ONNX file writer for the importer's tests (no `onnx` package here): the
protobuf wire format of the ModelProto fields a network file uses, written from the
published onnx.proto field numbers. Repeated integers are written unpacked, as proto2
serialisers do, except where `packed=True` asks for the packed form (both are legal)."""
import struct

import numpy as np


def varint(v):
    v &= (1 << 64) - 1
    out = bytearray()
    while True:
        b = v & 0x7F
        v >>= 7
        out.append(b | (0x80 if v else 0))
        if not v:
            return bytes(out)


def key(num, wt):
    return varint((num << 3) | wt)


def ld(num, payload):
    return key(num, 2) + varint(len(payload)) + payload


def s(num, text):
    return ld(num, text.encode())


def i(num, v):
    return key(num, 0) + varint(v)


def tensor(name, arr):
    arr = np.ascontiguousarray(arr)
    dt = {np.dtype(np.float32): 1, np.dtype(np.int32): 6, np.dtype(np.int64): 7}[arr.dtype]
    return b"".join(i(1, d) for d in arr.shape) + i(2, dt) + s(8, name) + ld(9, arr.tobytes())


def attr(name, v, packed=False):
    out = s(1, name)
    if isinstance(v, float):
        return out + key(2, 5) + struct.pack("<f", v) + i(20, 1)
    if isinstance(v, int):
        return out + i(3, v) + i(20, 2)
    if isinstance(v, str):
        return out + ld(4, v.encode()) + i(20, 3)
    if isinstance(v, np.ndarray):
        return out + ld(5, tensor("", v)) + i(20, 4)
    ints = [int(x) for x in v]
    body = ld(8, b"".join(varint(x) for x in ints)) if packed else b"".join(i(8, x) for x in ints)
    return out + body + i(20, 7)


def node(op, inputs, outputs, packed=False, **attrs):
    return (b"".join(s(1, n) for n in inputs) + b"".join(s(2, n) for n in outputs) +
            s(4, op) + b"".join(ld(5, attr(k, v, packed)) for k, v in attrs.items()))


def value_info(name, dims, elem=1):
    shape = b"".join(ld(1, i(1, d)) for d in dims)
    return s(1, name) + ld(2, ld(1, i(1, elem) + ld(2, shape)))


def model(nodes, initializers, inputs, outputs):
    """nodes: encoded NodeProtos; initializers: {name: array}; inputs / outputs:
    [(name, dims)]."""
    graph = (b"".join(ld(1, n) for n in nodes) + s(2, "g") +
             b"".join(ld(5, tensor(k, v)) for k, v in initializers.items()) +
             b"".join(ld(11, value_info(n, d)) for n, d in inputs) +
             b"".join(ld(12, value_info(n, d)) for n, d in outputs))
    return i(1, 8) + s(2, "pet-amd-tests") + ld(8, s(1, "") + i(2, 13)) + ld(7, graph)
