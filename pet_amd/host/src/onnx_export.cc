// GraphBase::exportOnnx: the operators of this graph -> an ONNX model file.
//
// The reference collects names, shapes and attributes per operator
// (src/Graph/graph.cc:1189-1340, Operator::getOptypeAttr, TransBasic::getOptypeDim) and hands
// them to its Python plug-in, which needs the `onnx` package to serialise them
// (python/cpp_plugin/export_onnx.py:71-227; weights are written as zeros there). Here the
// protobuf wire format is written directly (opset 17). An activation fused into a convolution
// or matmul becomes a node of its own, as upstream; a Transpose with a split or a merge
// becomes Reshape / Transpose / Reshape after its micro-op lowering; weights that hold data
// are written with it. What has no ONNX counterpart (ConvTrans in its NHWC form, G2BMM,
// GBMML, MemBound, a transpose with halo or padding parameters) makes the export fail with a
// message. Graph::importOnnx (onnx_import.cc) reads every file this writes.
#include "graph.h"
#include "transpose.h"

#include <cmath>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <map>
#include <stdexcept>
#include <string>
#include <tuple>
#include <vector>

namespace tpm {
namespace {

[[noreturn]] void fail(const std::string &what) { throw std::runtime_error(what); }

// ---------------------------------------------------------------- wire format

std::string varint(uint64_t v) {
    std::string out;
    do {
        uint8_t b = v & 0x7F;
        v >>= 7;
        out.push_back((char)(b | (v ? 0x80 : 0)));
    } while (v);
    return out;
}
std::string key(int num, int wt) { return varint(((uint64_t)num << 3) | (uint64_t)wt); }
std::string ld(int num, const std::string &payload) {
    return key(num, 2) + varint(payload.size()) + payload;
}
std::string vi(int num, int64_t v) { return key(num, 0) + varint((uint64_t)v); }

std::string floatTensor(const std::string &name, const Dim &dims, const VType *data, size_t n) {
    std::string t;
    for (int d : dims)
        t += vi(1, d);
    t += vi(2, 1) + ld(8, name);
    t += ld(9, std::string(reinterpret_cast<const char *>(data), n * sizeof(float)));
    return t;
}
std::string int64Tensor(const std::string &name, const std::vector<int64_t> &v,
                        const std::vector<int64_t> &dims) {
    std::string t;
    for (int64_t d : dims)
        t += vi(1, d);
    t += vi(2, 7) + ld(8, name);
    t += ld(9, std::string(reinterpret_cast<const char *>(v.data()), v.size() * 8));
    return t;
}

std::string attrInt(const std::string &name, int64_t v) { return ld(1, name) + vi(3, v) + vi(20, 2); }
std::string attrFloat(const std::string &name, float v) {
    uint32_t bits;
    std::memcpy(&bits, &v, 4);
    std::string raw(reinterpret_cast<const char *>(&bits), 4);
    return ld(1, name) + key(2, 5) + raw + vi(20, 1);
}
std::string attrInts(const std::string &name, const std::vector<int64_t> &v) {
    std::string a = ld(1, name);
    for (int64_t x : v)
        a += vi(8, x);
    return a + vi(20, 7);
}

std::string valueInfo(const std::string &name, const Dim &dims) {
    std::string shape;
    for (int d : dims)
        shape += ld(1, vi(1, d));
    const std::string tensorType = vi(1, 1) + ld(2, shape);
    return ld(1, name) + ld(2, ld(1, tensorType));
}

// ---------------------------------------------------------------- the graph

struct Exporter {
    std::string nodes, initializers;
    std::map<const Tensor *, std::string> names;
    std::map<std::string, bool> written; // initializers by name
    int counter = 0;

    std::string fresh(const char *stem) { return std::string(stem) + std::to_string(counter++); }

    std::string nameOf(const Tensor *t) {
        auto it = names.find(t);
        if (it != names.end())
            return it->second;
        const std::string n = "t" + std::to_string(names.size());
        names[t] = n;
        return n;
    }

    // A constant of the graph (weights, bias and normalisation vectors): written once
    std::string constant(Tensor *t, bool asIndices = false) {
        const std::string n = nameOf(t);
        if (written[n])
            return n;
        written[n] = true;
        const VType *data = t->getDataPtr(); // zeros when the tensor was never given values
        if (asIndices) {
            std::vector<int64_t> idx(t->size());
            for (size_t i = 0; i < idx.size(); ++i)
                idx[i] = (int64_t)std::llround(data[i]);
            std::vector<int64_t> dims(t->getDims().begin(), t->getDims().end());
            initializers += ld(5, int64Tensor(n, idx, dims));
        } else {
            initializers += ld(5, floatTensor(n, t->getDims(), data, t->size()));
        }
        return n;
    }

    std::string ints(const std::vector<int64_t> &v) {
        const std::string n = fresh("c");
        initializers += ld(5, int64Tensor(n, v, {(int64_t)v.size()}));
        return n;
    }

    void node(const std::string &op, const std::vector<std::string> &ins,
              const std::vector<std::string> &outs, const std::vector<std::string> &attrs = {}) {
        std::string n;
        for (auto &i : ins)
            n += ld(1, i);
        for (auto &o : outs)
            n += ld(2, o);
        n += ld(3, fresh((op + "_").c_str())) + ld(4, op);
        for (auto &a : attrs)
            n += ld(5, a);
        nodes += ld(1, n);
    }

    // an operand: a constant when it is a weight without a producer, else a named value
    std::string operand(Tensor *t, bool asIndices = false) {
        if (t->getOutputOf() == nullptr && t->getType() == Tensor::Weight)
            return constant(t, asIndices);
        return nameOf(t);
    }

    static const char *actName(Operator::ActType a) {
        switch (a) {
        case Operator::Relu:
            return "Relu";
        case Operator::Sigmoid:
            return "Sigmoid";
        case Operator::Tanh:
            return "Tanh";
        case Operator::Gelu:
            return "Gelu";
        default:
            return nullptr;
        }
    }

    // `produced` holds the value before the activation; the operator's output after it
    void finish(const std::string &produced, Tensor *out, Operator::ActType act) {
        if (const char *a = actName(act))
            node(a, {produced}, {nameOf(out)});
    }
    std::string before(Tensor *out, Operator::ActType act) {
        return actName(act) ? fresh("pre") : nameOf(out);
    }

    void transpose(TransposeOp *tr) {
        Tensor *in = tr->getInputs()[0], *out = tr->getOutputs()[0];
        std::vector<int> dims(in->getDims().begin(), in->getDims().end());
        std::string cur = operand(in);
        const auto micro = tr->getTTParam();
        if (micro.empty()) {
            node("Identity", {cur}, {nameOf(out)});
            return;
        }
        for (size_t i = 0; i < micro.size(); ++i) {
            std::vector<int> enc, perm;
            const size_t before = dimProduct(Dim(dims.begin(), dims.end()));
            if (!micro[i]->apply(dims, enc, perm))
                fail("a transpose whose lowering fails");
            const std::string dst = i + 1 == micro.size() ? nameOf(out) : fresh("tr");
            if (enc[0] == 1) {
                node("Transpose", {cur}, {dst},
                     {attrInts("perm", std::vector<int64_t>(perm.begin(), perm.end()))});
            } else {
                if (enc[2 + (enc[0] == 0)] != 0 || enc[3 + (enc[0] == 0)] != 0 ||
                    dimProduct(Dim(dims.begin(), dims.end())) != before)
                    fail("a transpose with halo or padding parameters has no ONNX form");
                node("Reshape", {cur, ints(std::vector<int64_t>(dims.begin(), dims.end()))}, {dst});
            }
            cur = dst;
        }
    }

    void op(Operator *o) {
        const TensorVec &in = o->getInputs(), &out = o->getOutputs();
        if (auto c = dynamic_cast<ConvOp *>(o)) {
            const Dim &w = in[1]->getDims(), &x = in[0]->getDims();
            std::vector<std::string> ins = {operand(in[0]), operand(in[1])};
            if (c->getBias())
                ins.push_back(constant(c->getBias()));
            const std::string pre = before(out[0], c->getAct());
            node("Conv", ins, {pre},
                 {attrInts("pads", {c->getPh(), c->getPw(), c->getPh(), c->getPw()}),
                  attrInts("strides", {c->getSh(), c->getSw()}),
                  attrInts("dilations", {c->getDh(), c->getDw()}),
                  attrInts("kernel_shape", {w[2], w[3]}), attrInt("group", x[1] / w[1])});
            finish(pre, out[0], c->getAct());
        } else if (auto c3 = dynamic_cast<Conv3dOp *>(o)) {
            const Dim &w = in[1]->getDims(), &x = in[0]->getDims();
            std::vector<std::string> ins = {operand(in[0]), operand(in[1])};
            if (c3->getBias())
                ins.push_back(constant(c3->getBias()));
            std::vector<int64_t> pads(c3->getPad().begin(), c3->getPad().end());
            pads.insert(pads.end(), c3->getPad().begin(), c3->getPad().end());
            const std::string pre = before(out[0], c3->getAct());
            node("Conv", ins, {pre},
                 {attrInts("pads", pads),
                  attrInts("strides", std::vector<int64_t>(c3->getStride().begin(), c3->getStride().end())),
                  attrInts("dilations",
                           std::vector<int64_t>(c3->getDilation().begin(), c3->getDilation().end())),
                  attrInts("kernel_shape", {w[2], w[3], w[4]}), attrInt("group", x[1] / w[1])});
            finish(pre, out[0], c3->getAct());
        } else if (auto m = dynamic_cast<MatmulOp *>(o)) {
            std::string a = operand(in[0]), b = operand(in[1]);
            if (m->getTransA()) {
                const std::string t = fresh("ta");
                node("Transpose", {a}, {t}, {attrInts("perm", {0, 2, 1})});
                a = t;
            }
            if (m->getTransB() && in[1]->getOutputOf() == nullptr &&
                in[1]->getType() == Tensor::Weight) {
                // a constant right-hand side is written transposed, under a name of its own
                const Dim &d = in[1]->getDims();
                const VType *src = in[1]->getDataPtr();
                std::vector<VType> tr(in[1]->size());
                for (int bi = 0; bi < d[0]; ++bi)
                    for (int r = 0; r < d[1]; ++r)
                        for (int c = 0; c < d[2]; ++c)
                            tr[((size_t)bi * d[2] + c) * d[1] + r] = src[((size_t)bi * d[1] + r) * d[2] + c];
                b = fresh("wt");
                initializers += ld(5, floatTensor(b, {d[0], d[2], d[1]}, tr.data(), tr.size()));
            } else if (m->getTransB()) {
                const std::string t = fresh("tb");
                node("Transpose", {b}, {t}, {attrInts("perm", {0, 2, 1})});
                b = t;
            }
            const std::string pre = before(out[0], m->getAct());
            if (m->getBias()) {
                const std::string mm = fresh("mm");
                node("MatMul", {a, b}, {mm});
                node("Add", {mm, constant(m->getBias())}, {pre});
            } else {
                node("MatMul", {a, b}, {pre});
            }
            finish(pre, out[0], m->getAct());
        } else if (auto tr = dynamic_cast<TransposeOp *>(o)) {
            transpose(tr);
        } else if (auto sp = dynamic_cast<SplitOp *>(o)) {
            std::vector<std::string> outs;
            std::vector<int64_t> sizes;
            for (auto t : out) {
                outs.push_back(nameOf(t));
                sizes.push_back(t->getDims()[sp->getDim()]);
            }
            node("Split", {operand(in[0]), ints(sizes)}, outs, {attrInt("axis", sp->getDim())});
        } else if (auto cc = dynamic_cast<ConcatOp *>(o)) {
            std::vector<std::string> ins;
            for (auto t : in)
                ins.push_back(operand(t));
            node("Concat", ins, {nameOf(out[0])}, {attrInt("axis", cc->getDim())});
        } else if (auto pd = dynamic_cast<PadOp *>(o)) {
            std::vector<int64_t> pads(pd->getBegin().begin(), pd->getBegin().end());
            pads.insert(pads.end(), pd->getEnd().begin(), pd->getEnd().end());
            node("Pad", {operand(in[0]), ints(pads)}, {nameOf(out[0])});
        } else if (auto sl = dynamic_cast<SliceOp *>(o)) {
            const Dim &d = in[0]->getDims();
            std::vector<int64_t> starts, ends, axes;
            for (size_t i = 0; i < d.size(); ++i) {
                starts.push_back(sl->getBegin()[i]);
                ends.push_back(d[i] - sl->getEnd()[i]);
                axes.push_back((int64_t)i);
            }
            node("Slice", {operand(in[0]), ints(starts), ints(ends), ints(axes)}, {nameOf(out[0])});
        } else if (auto ex = dynamic_cast<ExtendOp *>(o)) {
            std::vector<std::string> ins(ex->getNum() + 1, operand(in[0]));
            node("Concat", ins, {nameOf(out[0])}, {attrInt("axis", ex->getDim())});
        } else if (dynamic_cast<EltwiseOp *>(o)) {
            const char *name = o->getType() == Operator::Add   ? "Add"
                               : o->getType() == Operator::Sub ? "Sub"
                               : o->getType() == Operator::Mul ? "Mul"
                                                               : "Div";
            std::string acc = operand(in[0]);
            for (size_t i = 1; i < in.size(); ++i) {
                const std::string dst = i + 1 == in.size() ? nameOf(out[0]) : fresh("e");
                node(name, {acc, operand(in[i])}, {dst});
                acc = dst;
            }
            if (in.size() == 1)
                node("Identity", {acc}, {nameOf(out[0])});
        } else if (auto pw = dynamic_cast<PowOp *>(o)) {
            const std::string e = fresh("c");
            const VType p = (VType)pw->getPow();
            initializers += ld(5, floatTensor(e, {1}, &p, 1));
            node("Pow", {operand(in[0]), e}, {nameOf(out[0])});
        } else if (auto bn = dynamic_cast<BatchNormOp *>(o)) {
            node("BatchNormalization",
                 {operand(in[0]), constant(bn->getScale()), constant(bn->getBias()),
                  constant(bn->getMean()), constant(bn->getVar())},
                 {nameOf(out[0])}, {attrFloat("epsilon", bn->getEpsilon())});
        } else if (auto ga = dynamic_cast<GatherOp *>(o)) {
            node("Gather", {operand(in[0]), operand(in[1], true)}, {nameOf(out[0])},
                 {attrInt("axis", ga->getAxis())});
        } else if (auto rm = dynamic_cast<ReduceMeanOp *>(o)) {
            node("ReduceMean", {operand(in[0])}, {nameOf(out[0])},
                 {attrInts("axes", {rm->getAxis()}), attrInt("keepdims", 1)});
        } else if (auto ac = dynamic_cast<ActivationOp *>(o)) {
            const char *a = actName(ac->getActType());
            node(a ? a : "Identity", {operand(in[0])}, {nameOf(out[0])});
        } else if (auto pl = dynamic_cast<PoolOp *>(o)) {
            int kh, kw, ph, pw, sh, sw, dh, dw;
            std::tie(kh, kw, ph, pw, sh, sw, dh, dw) = pl->getArgs();
            if (dh != 1 || dw != 1)
                fail("dilated pooling has no counterpart in the reader");
            node(dynamic_cast<MaxPoolOp *>(o) ? "MaxPool" : "AveragePool", {operand(in[0])},
                 {nameOf(out[0])},
                 {attrInts("kernel_shape", {kh, kw}), attrInts("pads", {ph, pw, ph, pw}),
                  attrInts("strides", {sh, sw})});
        } else if (auto sm = dynamic_cast<SoftmaxOp *>(o)) {
            node("Softmax", {operand(in[0])}, {nameOf(out[0])}, {attrInt("axis", sm->getAxis())});
        } else if (auto ln = dynamic_cast<LayerNormOp *>(o)) {
            if (!ln->getGamma())
                fail("LayerNorm without a scale has no ONNX form");
            std::vector<std::string> ins = {operand(in[0]), constant(ln->getGamma())};
            if (ln->getBeta())
                ins.push_back(constant(ln->getBeta()));
            node("LayerNormalization", ins, {nameOf(out[0])},
                 {attrInt("axis", -1), attrFloat("epsilon", ln->getEps())});
        } else if (dynamic_cast<ReshapeOp *>(o)) { // Reshape, Identity, Flatten
            const Dim &d = out[0]->getDims();
            node("Reshape", {operand(in[0]), ints(std::vector<int64_t>(d.begin(), d.end()))},
                 {nameOf(out[0])});
        } else {
            fail(o->getName() + " has no ONNX counterpart");
        }
    }
};

} // namespace

bool GraphBase::exportOnnx(const char *path) {
    if (!path)
        return false;
    try {
        updateConnection();
        // the operators as they were added when that order is a topological one (it is for a
        // graph made by the builders), else sorted
        OpVec order = ops;
        std::map<const Operator *, size_t> position;
        for (size_t i = 0; i < order.size(); ++i)
            position[order[i]] = i;
        bool sorted = true;
        for (size_t i = 0; i < order.size() && sorted; ++i)
            for (auto t : order[i]->getInputs())
                if (t->getOutputOf() && position.count(t->getOutputOf()) &&
                    position[t->getOutputOf()] >= i)
                    sorted = false;
        if (!sorted) {
            order.clear();
            if (!topoOrder(order))
                fail("the graph has a cycle");
        }
        Exporter e;
        for (auto o : order)
            e.op(o);
        std::string graph = e.nodes + ld(2, "pet-optimization") + e.initializers;
        for (auto t : inputs)
            if (!(t->getOutputOf() == nullptr && t->getType() == Tensor::Weight))
                graph += ld(11, valueInfo(e.nameOf(t), t->getDims()));
        for (auto t : outputs)
            graph += ld(12, valueInfo(e.nameOf(t), t->getDims()));
        // ir_version 8, producer, the default operator set at version 17
        const std::string model =
            vi(1, 8) + ld(2, "PET") + ld(7, graph) + ld(8, ld(1, "") + vi(2, 17));
        std::ofstream f(path, std::ios::binary);
        f.write(model.data(), (std::streamsize)model.size());
        if (!f)
            fail("cannot write the file");
    } catch (const std::exception &ex) {
        std::fprintf(stderr, "[pet] exportOnnx(%s): %s\n", path, ex.what());
        return false;
    }
    return true;
}

} // namespace tpm
