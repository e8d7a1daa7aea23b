"""ONNX model files -> a Graph of the host layer, without the `onnx` package.

Role of the reference's python/cpp_plugin/import_onnx.py:125-459 (which needs `onnx`
for parsing and shape inference): the protobuf wire format is read directly (the
handful of ModelProto / GraphProto / NodeProto / AttributeProto / TensorProto /
ValueInfoProto fields a network file uses), and every operator is created through the
builder of `cpp_module.Graph` the reference's importer calls for it; output shapes
come from the builders' own shape rules instead of onnx.shape_inference.

    model = onnx_import.load("resnet18.onnx")
    sub, feeds = model.subgraph()       # weights uploaded; feeds: input name -> Tensor
    feeds["input"].setData(x); sub.compute(); y = sub.getOutputs()[0].getData()
"""
import struct

import numpy as np

FLOAT, INT32, INT64 = 1, 6, 7
_NP = {FLOAT: np.float32, INT32: np.int32, INT64: np.int64}


# ---------------------------------------------------------------- wire format

def _varint(buf, pos):
    val, shift = 0, 0
    while True:
        b = buf[pos]
        pos += 1
        val |= (b & 0x7F) << shift
        if not b & 0x80:
            return val, pos
        shift += 7


def _fields(buf):
    """(field number, wire type, value) of one message; value is an int for wire types
    0 / 1 / 5 (raw bits) and a memoryview for 2."""
    buf = memoryview(buf)
    pos, end = 0, len(buf)
    while pos < end:
        key, pos = _varint(buf, pos)
        num, wt = key >> 3, key & 7
        if wt == 0:
            val, pos = _varint(buf, pos)
        elif wt == 1:
            val, pos = struct.unpack_from("<Q", buf, pos)[0], pos + 8
        elif wt == 5:
            val, pos = struct.unpack_from("<I", buf, pos)[0], pos + 4
        elif wt == 2:
            n, pos = _varint(buf, pos)
            val, pos = buf[pos:pos + n], pos + n
        else:
            raise ValueError("unsupported protobuf wire type %d" % wt)
        yield num, wt, val


def _s64(v):
    return v - (1 << 64) if v >= 1 << 63 else v


def _ints(wt, val):
    """A repeated int64 field occurrence: packed (wire type 2) or a single varint."""
    if wt == 0:
        return [_s64(val)]
    out, pos = [], 0
    while pos < len(val):
        v, pos = _varint(val, pos)
        out.append(_s64(v))
    return out


def _floats(wt, val):
    if wt == 5:
        return [struct.unpack("<f", struct.pack("<I", val))[0]]
    return list(np.frombuffer(bytes(val), dtype="<f4"))


def _tensor(buf):
    dims, dtype, name, raw, f32, i32, i64 = [], FLOAT, "", None, [], [], []
    for num, wt, val in _fields(buf):
        if num == 1:
            dims += _ints(wt, val)
        elif num == 2:
            dtype = val
        elif num == 4:
            f32 += _floats(wt, val)
        elif num == 5:
            i32 += _ints(wt, val)
        elif num == 7:
            i64 += _ints(wt, val)
        elif num == 8:
            name = bytes(val).decode()
        elif num == 9:
            raw = bytes(val)
    if dtype not in _NP:
        raise ValueError("tensor %r has unsupported data type %d" % (name, dtype))
    if raw is not None:
        data = np.frombuffer(raw, dtype=np.dtype(_NP[dtype]).newbyteorder("<"))
    else:
        data = np.array({FLOAT: f32, INT32: i32, INT64: i64}[dtype], dtype=_NP[dtype])
    return name, data.astype(_NP[dtype]).reshape(dims)


def _attribute(buf):
    name, out, ints, floats = "", None, [], []
    for num, wt, val in _fields(buf):
        if num == 1:
            name = bytes(val).decode()
        elif num == 2:
            out = _floats(wt, val)[0]
        elif num == 3:
            out = _s64(val)
        elif num == 4:
            out = bytes(val).decode()
        elif num == 5:
            out = _tensor(val)[1]
        elif num == 7:
            floats += _floats(wt, val)
        elif num == 8:
            ints += _ints(wt, val)
    if ints:
        out = ints
    elif floats:
        out = floats
    return name, out


def _value_info(buf):
    name, dims, elem = "", [], FLOAT
    for num, _, val in _fields(buf):
        if num == 1:
            name = bytes(val).decode()
        elif num == 2:                                    # TypeProto
            for n2, _, v2 in _fields(val):
                if n2 == 1:                               # tensor_type
                    for n3, _, v3 in _fields(v2):
                        if n3 == 1:
                            elem = v3
                        elif n3 == 2:                     # TensorShapeProto
                            for n4, _, v4 in _fields(v3):
                                if n4 == 1:               # Dimension
                                    d = 0
                                    for n5, _, v5 in _fields(v4):
                                        if n5 == 1:
                                            d = _s64(v5)
                                    dims.append(d)
    return name, dims, elem


class Node:
    def __init__(self, buf):
        self.inputs, self.outputs, self.op, self.name, self.attrs = [], [], "", "", {}
        for num, _, val in _fields(buf):
            if num == 1:
                self.inputs.append(bytes(val).decode())
            elif num == 2:
                self.outputs.append(bytes(val).decode())
            elif num == 3:
                self.name = bytes(val).decode()
            elif num == 4:
                self.op = bytes(val).decode()
            elif num == 5:
                k, v = _attribute(val)
                self.attrs[k] = v


def parse(data):
    """-> (nodes, initializers {name: array}, inputs [(name, dims)], outputs [names])."""
    graph = None
    for num, wt, val in _fields(data):
        if num == 7 and wt == 2:
            graph = val
    if graph is None:
        raise ValueError("no graph in the model file")
    nodes, inits, inputs, outputs = [], {}, [], []
    for num, _, val in _fields(graph):
        if num == 1:
            nodes.append(Node(val))
        elif num == 5:
            name, arr = _tensor(val)
            inits[name] = arr
        elif num == 11:
            name, dims, _ = _value_info(val)
            inputs.append((name, dims))
        elif num == 12:
            outputs.append(_value_info(val)[0])
    return nodes, inits, inputs, outputs


# ---------------------------------------------------------------- graph building

class Model:
    def __init__(self, module, graph):
        self.module, self.graph = module, graph
        self.tensors, self.weights, self.inputs, self.outputs = {}, {}, [], []

    def subgraph(self):
        """SubGraph of the whole model with the weights' data in place; returns it and
        {input name: its Tensor in the SubGraph}."""
        self.graph.updateConnection()
        # bias / batch-norm vectors are side pointers of their operators: the copies of
        # the operators in the SubGraph keep pointing at this graph's tensors
        for name, arr in self.weights.items():
            self.tensors[name].setData(arr.astype(np.float32))
        sub = self.module.SubGraph(self.graph.getOperators())
        sub.model = self    # the side tensors live in self.graph: keep it alive with the SubGraph
        by_hash = {self.tensors[n].getHash(): n for n in list(self.weights) + self.inputs}
        feeds = {}
        for t in sub.getInputs():
            name = by_hash.get(t.getHash())
            if name in self.weights:
                t.setData(self.weights[name].astype(np.float32))
            elif name is not None:
                feeds[name] = t
        return sub, feeds


def _module():
    import glob
    import importlib
    import os
    import sys
    lib = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")
    if not glob.glob(os.path.join(lib, "cpp_module*.so")):
        raise ImportError("pet_amd/lib/cpp_module*.so is not built (make -C pet_amd/host)")
    if lib not in sys.path:
        sys.path.insert(0, lib)
    return importlib.import_module("cpp_module")


def _sym(pads, n):
    pads = list(pads) if pads else [0] * (2 * n)
    if pads[:n] != pads[n:]:
        raise ValueError("asymmetric padding %s" % (pads,))
    return pads[:n]


def fold_batchnorm(nodes, inits, outputs):
    """Conv -> BatchNormalization with constant parameters, the convolution's result used
    nowhere else: the normalisation goes into the filters and the bias (what exporters
    do when they "fold BN"; the benchmark's ResNets are stated that way). Returns the new
    node list; new initializers are added to `inits`."""
    users = {}
    for nd in nodes:
        for n in nd.inputs:
            users[n] = users.get(n, 0) + 1
    by_out = {nd.outputs[0]: nd for nd in nodes if nd.outputs}
    dropped, out_nodes = set(), []
    for nd in nodes:
        if nd.op != "BatchNormalization" or any(n not in inits for n in nd.inputs[1:5]):
            continue
        conv = by_out.get(nd.inputs[0])
        if (conv is None or conv.op != "Conv" or users.get(conv.outputs[0], 0) != 1 or
                conv.outputs[0] in outputs or any(n not in inits for n in conv.inputs[1:])):
            continue
        sc, bi, me, va = (inits[n].astype(np.float64) for n in nd.inputs[1:5])
        factor = sc / np.sqrt(va + float(nd.attrs.get("epsilon", 1e-5)))
        w = inits[conv.inputs[1]].astype(np.float64)
        b = inits[conv.inputs[2]].astype(np.float64) if len(conv.inputs) > 2 else np.zeros(w.shape[0])
        wn, bn = conv.inputs[1] + "::bn", conv.outputs[0] + "::bn_bias"
        inits[wn] = (w * factor.reshape((-1,) + (1,) * (w.ndim - 1))).astype(np.float32)
        inits[bn] = ((b - me) * factor + bi).astype(np.float32)
        conv.inputs = [conv.inputs[0], wn, bn]
        conv.outputs = [nd.outputs[0]]
        dropped.add(id(nd))
    for nd in nodes:
        if id(nd) not in dropped:
            out_nodes.append(nd)
    return out_nodes


def load(source, module=None, fold_bn=True):
    """source: a path or the bytes of an ONNX file. fold_bn: BatchNormalization after a
    convolution with constant parameters is folded into that convolution."""
    cm = module or _module()
    data = source if isinstance(source, (bytes, bytearray, memoryview)) else open(source, "rb").read()
    nodes, inits, inputs, outputs = parse(data)
    if fold_bn:
        nodes = fold_batchnorm(nodes, inits, outputs)
    g = cm.Graph()
    m = Model(cm, g)
    const = dict(inits)                         # values known at import time

    def new(dims):
        return g.tensor([int(d) for d in dims], "FLOAT")

    for name, dims in inputs:
        if name not in inits:
            if any(d <= 0 for d in dims):
                raise ValueError("input %r has a symbolic shape %s" % (name, dims))
            m.tensors[name] = new(dims)
            m.inputs.append(name)

    def weight(name):
        if name not in m.tensors:
            arr = const[name]
            t = new(arr.shape if arr.ndim else [1])
            t.setWeight()
            m.tensors[name] = t
            m.weights[name] = np.ascontiguousarray(arr, dtype=np.float32).reshape(t.getDims())
        return m.tensors[name]

    def tin(name):
        return m.tensors[name] if name in m.tensors else weight(name)

    def same_shape(x):
        return new(x.getDims())

    for nd in nodes:
        a, op = nd.attrs, nd.op
        ins = [n for n in nd.inputs]
        out = None
        if op in ("Constant",):
            const[nd.outputs[0]] = np.asarray(a["value"])
            continue
        if op == "Shape":
            const[nd.outputs[0]] = np.array(tin(ins[0]).getDims(), dtype=np.int64)
            continue
        x = tin(ins[0])
        xd = x.getDims()
        if op == "Conv":
            w = tin(ins[1])
            bias = tin(ins[2]) if len(ins) > 2 else None
            nsp = len(xd) - 2
            pads = _sym(a.get("pads"), nsp)
            st = list(a.get("strides", [1] * nsp))
            dil = list(a.get("dilations", [1] * nsp))
            if a.get("auto_pad", "NOTSET") != "NOTSET":
                raise ValueError("auto_pad is not supported")
            if nsp == 2:
                out = g.conv(x, w, pads[0], pads[1], st[0], st[1], dil[0], dil[1], bias).getOutput()
            elif nsp == 3:
                wd = w.getDims()
                od = [xd[0], wd[0]] + [(xd[2 + i] + 2 * pads[i] - dil[i] * (wd[2 + i] - 1) - 1)
                                       // st[i] + 1 for i in range(3)]
                out = new(od)
                g.conv3d(x, w, out, pads, st, dil, bias)
            else:
                raise ValueError("Conv with %d spatial dims" % nsp)
        elif op in ("Relu", "Sigmoid", "Tanh", "Gelu", "Identity", "Cast", "Dropout"):
            if op == "Gelu" and a.get("approximate", "none") != "none":
                raise ValueError("Gelu: the exact form only")
            out = same_shape(x)
            {"Relu": g.relu, "Sigmoid": g.sigmoid, "Tanh": g.tanh, "Gelu": g.gelu}.get(
                op, g.identity)(x, out)
        elif op in ("Add", "Mul", "Sub", "Div"):
            y = tin(ins[1])
            big, small = (x, y) if x.size() >= y.size() else (y, x)
            bd, sd = big.getDims(), [d for d in small.getDims()]
            while len(sd) > 1 and sd[0] == 1:
                sd = sd[1:]
            if sd != bd[len(bd) - len(sd):] and small.size() != 1:
                raise ValueError("%s: only trailing-dimension broadcast is supported (%s, %s)"
                                 % (op, bd, small.getDims()))
            out = new(bd)
            if op == "Add":
                g.add([x, y], out)
            elif op == "Mul":
                g.mul([x, y], out)
            elif op == "Sub":
                g.sub(x, y, out)
            else:
                g.div(x, y, out)
        elif op in ("MaxPool", "AveragePool"):
            k = list(a["kernel_shape"])
            pads = _sym(a.get("pads"), 2)
            st = list(a.get("strides", [1, 1]))
            if a.get("ceil_mode", 0) or len(k) != 2:
                raise ValueError("%s: ceil_mode / non-2-D pooling is not supported" % op)
            # the backend's average leaves padding out of the divisor (ONNX's default,
            # and the reference's cuDNN mode); max pooling is built without dilation
            if op == "AveragePool" and int(a.get("count_include_pad", 0)) and any(pads):
                raise ValueError("AveragePool: count_include_pad=1 with padding is not supported")
            if any(int(d) != 1 for d in a.get("dilations", [1, 1])):
                raise ValueError("%s: dilated pooling is not supported" % op)
            od = xd[:2] + [(xd[2 + i] + 2 * pads[i] - k[i]) // st[i] + 1 for i in range(2)]
            out = new(od)
            if op == "MaxPool":
                g.maxpool(x, out, k[0], k[1], 1, 1, pads[0], pads[1], st[0], st[1])
            else:
                g.avgpool(x, out, k[0], k[1], pads[0], pads[1], st[0], st[1])
        elif op == "GlobalAveragePool":
            out = new(xd[:2] + [1] * (len(xd) - 2))
            g.avgpool(x, out)
        elif op == "BatchNormalization":
            sc, bi, me, va = (tin(n) for n in ins[1:5])
            out = g.batchnorm(x, sc, bi, me, va, float(a.get("epsilon", 1e-5)), 0.9).getOutput()
        elif op == "MatMul":
            out = g.matmul(x, tin(ins[1])).getOutput()
        elif op == "Gemm":
            if float(a.get("alpha", 1.0)) != 1.0 or float(a.get("beta", 1.0)) != 1.0:
                raise ValueError("Gemm with alpha / beta other than 1")
            bias = tin(ins[2]) if len(ins) > 2 else None
            y = tin(ins[1])
            n_out = y.getDims()[0] if a.get("transB", 0) else y.getDims()[-1]
            if bias is not None and bias.size() != n_out:
                raise ValueError("Gemm: C must be a vector of the output's last dim")
            out = g.matmul(x, y, bool(a.get("transA", 0)), bool(a.get("transB", 0)), bias).getOutput()
        elif op == "Flatten":
            ax = int(a.get("axis", 1))
            out = new([int(np.prod(xd[:ax], dtype=np.int64)), int(np.prod(xd[ax:], dtype=np.int64))])
            g.flatten(x, out, ax)
        elif op == "Reshape":
            shape = [int(v) for v in np.asarray(const[ins[1]]).reshape(-1)]
            shape = [xd[i] if v == 0 else v for i, v in enumerate(shape)]
            if -1 in shape:
                known = int(np.prod([v for v in shape if v != -1], dtype=np.int64))
                shape[shape.index(-1)] = x.size() // max(known, 1)
            out = new(shape)
            g.reshape(x, out)
        elif op == "Transpose":
            perm = list(a.get("perm", range(len(xd) - 1, -1, -1)))
            out = g.transpose(x, -1, [int(p) for p in perm], 2).getOutput()
        elif op == "Concat":
            ax = int(a["axis"]) % len(xd)
            out = g.concat([tin(n) for n in ins], ax).getOutput()
        elif op == "Split":
            ax = int(a.get("axis", 0)) % len(xd)
            sizes = a.get("split") or (const[ins[1]].tolist() if len(ins) > 1 else
                                       [xd[ax] // len(nd.outputs)] * len(nd.outputs))
            outs = g.split(x, ax, [int(v) for v in sizes]).getOutputs()
            for name, t in zip(nd.outputs, outs):
                m.tensors[name] = t
            continue
        elif op == "Softmax":
            ax = int(a.get("axis", -1)) % len(xd)
            if ax != len(xd) - 1:
                raise ValueError("Softmax over an axis other than the last")
            out = same_shape(x)
            g.softmax(x, out, ax)
        elif op == "LayerNormalization":
            if int(a.get("axis", -1)) % len(xd) != len(xd) - 1:
                raise ValueError("LayerNormalization over more than the last axis")
            out = same_shape(x)
            g.layernorm(x, out, tin(ins[1]), tin(ins[2]) if len(ins) > 2 else None,
                        float(a.get("epsilon", 1e-5)))
        elif op == "Gather":
            idx = tin(ins[1])
            out = g.gather(x, idx, int(a.get("axis", 0)) % len(xd)).getOutput()
        elif op == "ReduceMean":
            axes = a.get("axes") or const[ins[1]].tolist()
            if len(axes) != 1 or not a.get("keepdims", 1):
                raise ValueError("ReduceMean over one axis with keepdims only")
            out = g.reduceMean(x, int(axes[0]) % len(xd)).getOutput()
        elif op == "Pad":
            pads = a.get("pads") or const[ins[1]].tolist()
            if a.get("mode", "constant") != "constant":
                raise ValueError("Pad: constant mode only")
            r = len(xd)
            out = g.pad(x, [int(p) for p in pads[:r]], [int(p) for p in pads[r:]]).getOutput()
        elif op == "Slice":
            lists = [np.asarray(const[n]).reshape(-1).tolist() if n else []
                     for n in list(ins[1:5]) + [""] * (5 - len(ins))]
            starts, ends, axes, steps = lists
            axes = axes or list(range(len(starts)))
            if not starts or not (len(starts) == len(ends) == len(axes)) or \
                    len(set(int(ax) % len(xd) for ax in axes)) != len(axes):
                raise ValueError("Slice: starts, ends and axes of different lengths")
            if any(st != 1 for st in steps):
                raise ValueError("Slice with a step other than 1")
            begin, drop = [0] * len(xd), [0] * len(xd)
            for lo, hi, ax in zip(starts, ends, axes):
                ax = int(ax) % len(xd)
                n = xd[ax]
                lo = min(max(lo + n if lo < 0 else lo, 0), n)
                hi = min(max(hi + n if hi < 0 else hi, 0), n)
                if hi <= lo:
                    raise ValueError("Slice: an empty range")
                begin[ax], drop[ax] = int(lo), int(n - hi)
            out = g.slice(x, begin, drop).getOutput()
        elif op == "Pow":
            p = float(np.asarray(const[ins[1]]).reshape(-1)[0])
            if p != int(p) or p < 0:
                raise ValueError("Pow with a non-integer exponent")
            out = g.pow(x, int(p)).getOutput()
        else:
            raise ValueError("ONNX operator %s is not supported" % op)
        m.tensors[nd.outputs[0]] = out
    m.outputs = list(outputs)
    g.updateConnection()
    return m
