// GraphBase::importOnnx: an ONNX model file -> operators of this Graph.
//
// The reference hands the file to its embedded Python plug-in
// (src/Graph/graph.cc:1172-1187 -> python/cpp_plugin/import_onnx.py:125-459, which needs the
// `onnx` package for parsing and shape inference). Here the protobuf wire format is read
// directly (the ModelProto / GraphProto / NodeProto / AttributeProto / TensorProto /
// ValueInfoProto fields a network file uses) and every node goes through the same Graph
// builder the plug-in calls for it; output shapes come from the builders' own shape rules.
// BatchNormalization behind a convolution with constant parameters is folded into that
// convolution's filters and bias. The Python front end (pet_amd/onnx_import.py) follows the
// same rules and is tested against this one.
#include "graph.h"

#include <cmath>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <map>
#include <set>
#include <stdexcept>
#include <string>
#include <vector>

namespace tpm {
namespace {

[[noreturn]] void fail(const std::string &what) { throw std::runtime_error(what); }

// ---------------------------------------------------------------- wire format

struct Reader {
    const uint8_t *p, *end;
};

uint64_t varint(Reader &r) {
    uint64_t v = 0;
    for (int shift = 0; shift < 70; shift += 7) {
        if (r.p >= r.end)
            fail("truncated varint");
        const uint8_t b = *r.p++;
        v |= (uint64_t)(b & 0x7F) << shift;
        if (!(b & 0x80))
            return v;
    }
    fail("varint longer than 10 bytes");
}

struct Field {
    uint32_t num = 0;
    int wt = 0;
    uint64_t val = 0;              // wire types 0, 1, 5 (raw bits)
    Reader sub{nullptr, nullptr};  // wire type 2
};

bool next(Reader &r, Field &f) {
    if (r.p >= r.end)
        return false;
    const uint64_t key = varint(r);
    f.num = (uint32_t)(key >> 3);
    f.wt = (int)(key & 7);
    switch (f.wt) {
    case 0:
        f.val = varint(r);
        break;
    case 1:
        if (r.end - r.p < 8)
            fail("truncated 64-bit field");
        std::memcpy(&f.val, r.p, 8);
        r.p += 8;
        break;
    case 5: {
        if (r.end - r.p < 4)
            fail("truncated 32-bit field");
        uint32_t v;
        std::memcpy(&v, r.p, 4);
        f.val = v;
        r.p += 4;
        break;
    }
    case 2: {
        const uint64_t n = varint(r);
        if ((uint64_t)(r.end - r.p) < n)
            fail("truncated length-delimited field");
        f.sub = Reader{r.p, r.p + n};
        r.p += n;
        break;
    }
    default:
        fail("unsupported protobuf wire type " + std::to_string(f.wt));
    }
    return true;
}

std::string text(const Reader &r) { return std::string((const char *)r.p, r.end - r.p); }

// one occurrence of a repeated int64 field: packed (wire type 2) or a single varint
void ints(const Field &f, std::vector<int64_t> &out) {
    if (f.wt == 0) {
        out.push_back((int64_t)f.val);
        return;
    }
    Reader r = f.sub;
    while (r.p < r.end)
        out.push_back((int64_t)varint(r));
}

void floats(const Field &f, std::vector<float> &out) {
    if (f.wt == 5) {
        const uint32_t bits = (uint32_t)f.val;
        float v;
        std::memcpy(&v, &bits, 4);
        out.push_back(v);
        return;
    }
    const size_t n = (f.sub.end - f.sub.p) / 4;
    const size_t at = out.size();
    out.resize(at + n);
    std::memcpy(out.data() + at, f.sub.p, n * 4);
}

enum { kFloat = 1, kInt32 = 6, kInt64 = 7 };

// A constant: values kept as doubles (exact for float32, int32 and the int64 a model uses
// for shapes, axes and indices)
struct Array {
    std::vector<int64_t> dims;
    std::vector<double> v;
    bool integral = false;
    size_t size() const { return v.size(); }
};

Array tensorProto(Reader r, std::string &name) {
    Array a;
    int dtype = kFloat;
    std::vector<float> f32;
    std::vector<int64_t> i32, i64;
    Reader raw{nullptr, nullptr};
    bool hasRaw = false;
    Field f;
    while (next(r, f)) {
        if (f.num == 1)
            ints(f, a.dims);
        else if (f.num == 2)
            dtype = (int)f.val;
        else if (f.num == 4)
            floats(f, f32);
        else if (f.num == 5)
            ints(f, i32);
        else if (f.num == 7)
            ints(f, i64);
        else if (f.num == 8)
            name = text(f.sub);
        else if (f.num == 9) {
            raw = f.sub;
            hasRaw = true;
        }
    }
    if (dtype != kFloat && dtype != kInt32 && dtype != kInt64)
        fail("tensor " + name + " has unsupported data type " + std::to_string(dtype));
    a.integral = dtype != kFloat;
    if (hasRaw) {
        const size_t bytes = raw.end - raw.p, w = dtype == kInt64 ? 8 : 4;
        a.v.resize(bytes / w);
        for (size_t i = 0; i < a.v.size(); ++i) {
            if (dtype == kFloat) {
                float x;
                std::memcpy(&x, raw.p + 4 * i, 4);
                a.v[i] = x;
            } else if (dtype == kInt32) {
                int32_t x;
                std::memcpy(&x, raw.p + 4 * i, 4);
                a.v[i] = x;
            } else {
                int64_t x;
                std::memcpy(&x, raw.p + 8 * i, 8);
                a.v[i] = (double)x;
            }
        }
    } else if (dtype == kFloat) {
        a.v.assign(f32.begin(), f32.end());
    } else {
        const std::vector<int64_t> &src = dtype == kInt32 ? i32 : i64;
        a.v.assign(src.begin(), src.end());
    }
    size_t want = 1;
    for (int64_t d : a.dims)
        want *= (size_t)d;
    if (want != a.v.size())
        fail("tensor " + name + ": " + std::to_string(a.v.size()) + " values for a shape of " +
             std::to_string(want));
    return a;
}

struct Attr {
    enum Kind { None, Float, Int, String, Tensor, Ints, Floats } kind = None;
    double f = 0;
    int64_t i = 0;
    std::string s;
    Array t;
    std::vector<int64_t> is;
    std::vector<float> fs;
};

Attr attributeProto(Reader r, std::string &name) {
    Attr a;
    Field f;
    while (next(r, f)) {
        if (f.num == 1) {
            name = text(f.sub);
        } else if (f.num == 2) {
            std::vector<float> one;
            floats(f, one);
            a.kind = Attr::Float;
            a.f = one.empty() ? 0 : one[0];
        } else if (f.num == 3) {
            a.kind = Attr::Int;
            a.i = (int64_t)f.val;
        } else if (f.num == 4) {
            a.kind = Attr::String;
            a.s = text(f.sub);
        } else if (f.num == 5) {
            std::string ignored;
            a.kind = Attr::Tensor;
            a.t = tensorProto(f.sub, ignored);
        } else if (f.num == 7) {
            floats(f, a.fs);
        } else if (f.num == 8) {
            ints(f, a.is);
        }
    }
    if (!a.is.empty())
        a.kind = Attr::Ints;
    else if (!a.fs.empty())
        a.kind = Attr::Floats;
    return a;
}

struct ValueInfo {
    std::string name;
    std::vector<int64_t> dims;
};

ValueInfo valueInfoProto(Reader r) {
    ValueInfo vi;
    Field f, f2, f3, f4, f5;
    while (next(r, f)) {
        if (f.num == 1) {
            vi.name = text(f.sub);
        } else if (f.num == 2) { // TypeProto
            Reader r2 = f.sub;
            while (next(r2, f2)) {
                if (f2.num != 1) // tensor_type
                    continue;
                Reader r3 = f2.sub;
                while (next(r3, f3)) {
                    if (f3.num != 2) // TensorShapeProto
                        continue;
                    Reader r4 = f3.sub;
                    while (next(r4, f4)) {
                        if (f4.num != 1) // Dimension
                            continue;
                        int64_t d = 0;
                        Reader r5 = f4.sub;
                        while (next(r5, f5))
                            if (f5.num == 1)
                                d = (int64_t)f5.val;
                        vi.dims.push_back(d);
                    }
                }
            }
        }
    }
    return vi;
}

struct Node {
    std::vector<std::string> inputs, outputs;
    std::string name, op;
    std::map<std::string, Attr> attrs;

    bool has(const char *k) const { return attrs.count(k) != 0; }
    int64_t geti(const char *k, int64_t dflt) const {
        auto it = attrs.find(k);
        return it == attrs.end() ? dflt : it->second.i;
    }
    double getf(const char *k, double dflt) const {
        auto it = attrs.find(k);
        return it == attrs.end() ? dflt : it->second.f;
    }
    std::string gets(const char *k, const char *dflt) const {
        auto it = attrs.find(k);
        return it == attrs.end() ? std::string(dflt) : it->second.s;
    }
    std::vector<int64_t> getis(const char *k) const {
        auto it = attrs.find(k);
        return it == attrs.end() ? std::vector<int64_t>() : it->second.is;
    }
};

Node nodeProto(Reader r) {
    Node n;
    Field f;
    while (next(r, f)) {
        if (f.num == 1)
            n.inputs.push_back(text(f.sub));
        else if (f.num == 2)
            n.outputs.push_back(text(f.sub));
        else if (f.num == 3)
            n.name = text(f.sub);
        else if (f.num == 4)
            n.op = text(f.sub);
        else if (f.num == 5) {
            std::string k;
            Attr a = attributeProto(f.sub, k);
            n.attrs[k] = a;
        }
    }
    return n;
}

struct Model {
    std::vector<Node> nodes;
    std::map<std::string, Array> inits;
    std::vector<ValueInfo> inputs;
    std::vector<std::string> outputs;
};

Model parse(const std::vector<uint8_t> &data) {
    Reader r{data.data(), data.data() + data.size()};
    Reader graph{nullptr, nullptr};
    Field f;
    while (next(r, f))
        if (f.num == 7 && f.wt == 2)
            graph = f.sub;
    if (!graph.p)
        fail("no graph in the model file");
    Model m;
    while (next(graph, f)) {
        if (f.wt != 2)
            continue;
        if (f.num == 1) {
            m.nodes.push_back(nodeProto(f.sub));
        } else if (f.num == 5) {
            std::string name;
            Array a = tensorProto(f.sub, name);
            m.inits[name] = a;
        } else if (f.num == 11) {
            m.inputs.push_back(valueInfoProto(f.sub));
        } else if (f.num == 12) {
            m.outputs.push_back(valueInfoProto(f.sub).name);
        }
    }
    return m;
}

// Conv -> BatchNormalization with constant parameters, the convolution's result used
// nowhere else: the normalisation goes into the filters and the bias.
void foldBatchnorm(Model &m) {
    std::map<std::string, int> users;
    for (auto &nd : m.nodes)
        for (auto &n : nd.inputs)
            ++users[n];
    std::map<std::string, Node *> byOut;
    for (auto &nd : m.nodes)
        if (!nd.outputs.empty())
            byOut[nd.outputs[0]] = &nd;
    std::set<const Node *> dropped;
    const std::set<std::string> outs(m.outputs.begin(), m.outputs.end());
    for (auto &nd : m.nodes) {
        if (nd.op != "BatchNormalization" || nd.inputs.size() < 5 || nd.outputs.empty())
            continue;
        bool constant = true;
        for (int i = 1; i < 5; ++i)
            constant = constant && m.inits.count(nd.inputs[i]);
        auto it = byOut.find(nd.inputs[0]);
        if (!constant || it == byOut.end())
            continue;
        Node *conv = it->second;
        if (conv->op != "Conv" || conv->inputs.size() < 2 || users[conv->outputs[0]] != 1 ||
            outs.count(conv->outputs[0]))
            continue;
        bool convConst = true;
        for (size_t i = 1; i < conv->inputs.size(); ++i)
            convConst = convConst && m.inits.count(conv->inputs[i]);
        if (!convConst)
            continue;
        const Array &sc = m.inits[nd.inputs[1]], &bi = m.inits[nd.inputs[2]],
                    &me = m.inits[nd.inputs[3]], &va = m.inits[nd.inputs[4]];
        const double eps = nd.getf("epsilon", 1e-5);
        Array w = m.inits[conv->inputs[1]];
        if (w.dims.empty() || w.dims[0] < 1 || w.size() % (size_t)w.dims[0] != 0)
            continue;
        const size_t F = (size_t)w.dims[0], per = w.size() / F;
        if (sc.size() != F || bi.size() != F || me.size() != F || va.size() != F ||
            (conv->inputs.size() > 2 && m.inits[conv->inputs[2]].size() != F))
            continue;
        Array b;
        b.dims = {(int64_t)F};
        b.v.assign(F, 0.0);
        if (conv->inputs.size() > 2)
            b.v = m.inits[conv->inputs[2]].v;
        for (size_t f = 0; f < F; ++f) {
            const double factor = sc.v[f] / std::sqrt(va.v[f] + eps);
            for (size_t i = 0; i < per; ++i)
                w.v[f * per + i] = (double)(float)(w.v[f * per + i] * factor);
            b.v[f] = (double)(float)((b.v[f] - me.v[f]) * factor + bi.v[f]);
        }
        const std::string wn = conv->inputs[1] + "::bn", bn = conv->outputs[0] + "::bn_bias";
        m.inits[wn] = w;
        m.inits[bn] = b;
        conv->inputs = {conv->inputs[0], wn, bn};
        conv->outputs = {nd.outputs[0]};
        dropped.insert(&nd);
    }
    std::vector<Node> kept;
    for (auto &nd : m.nodes)
        if (!dropped.count(&nd))
            kept.push_back(nd);
    m.nodes.swap(kept);
}

// ---------------------------------------------------------------- graph building

Dim checkedDims(const std::vector<int64_t> &dims, const std::string &what) {
    Dim out;
    long long total = 1;
    for (int64_t d : dims) {
        if (d < 1 || d >= (1ll << 31) || (total *= d) >= (1ll << 31))
            fail(what + ": a shape this backend does not take");
        out.push_back((int)d);
    }
    if (out.size() > 8)
        fail(what + ": more than 8 dims");
    return out;
}

struct Builder {
    Graph *g;
    std::map<std::string, Tensor *> tensors;
    std::map<std::string, Array> consts; // values known at import time

    Tensor *fresh(const Dim &dims) { return g->tensor(dims); }

    Tensor *weight(const std::string &name) {
        auto it = tensors.find(name);
        if (it != tensors.end())
            return it->second;
        auto c = consts.find(name);
        if (c == consts.end())
            fail("tensor " + name + " is neither computed nor a constant");
        Dim dims = checkedDims(c->second.dims, "constant " + name);
        if (dims.empty())
            dims.push_back(1);
        Tensor *t = g->tensor(dims);
        t->setType(Tensor::Weight);
        if (t->size() != c->second.v.size())
            fail("constant " + name + " holds " + std::to_string(c->second.v.size()) +
                 " values for " + std::to_string(t->size()));
        std::vector<VType> host(c->second.v.begin(), c->second.v.end());
        if (!t->setData(host.data())) // host side; uploaded when an operator first needs it
            fail("cannot keep the values of " + name);
        tensors[name] = t;
        return t;
    }

    Tensor *in(const std::string &name) { return weight(name); }

    const Array &constant(const std::string &name) {
        auto c = consts.find(name);
        if (c == consts.end())
            fail("the value of " + name + " is not known at import time");
        return c->second;
    }
};

std::vector<int> symmetricPads(const Node &nd, int n) {
    std::vector<int64_t> pads = nd.getis("pads");
    if (pads.empty())
        pads.assign(2 * n, 0);
    if ((int)pads.size() != 2 * n)
        fail(nd.op + ": " + std::to_string(pads.size()) + " pads for " + std::to_string(n) + " dims");
    std::vector<int> out;
    for (int i = 0; i < n; ++i) {
        if (pads[i] != pads[i + n])
            fail(nd.op + ": asymmetric padding");
        if (pads[i] < 0 || pads[i] > (1 << 20))
            fail(nd.op + ": padding of " + std::to_string(pads[i]));
        out.push_back((int)pads[i]);
    }
    return out;
}

std::vector<int> intsOr(const Node &nd, const char *key, int n, int dflt) {
    std::vector<int64_t> v = nd.getis(key);
    std::vector<int> out(n, dflt);
    for (int i = 0; i < n && i < (int)v.size(); ++i) {
        if (v[i] < 1 || v[i] > (1 << 20))
            fail(nd.op + ": " + key + " of " + std::to_string(v[i]));
        out[i] = (int)v[i];
    }
    return out;
}


Tensor *resultOf(Operator *op) { return op ? op->getOutput() : nullptr; }

void build(Graph *g, Model &m) {
    Builder b{g, {}, m.inits};
    for (auto &vi : m.inputs) {
        if (m.inits.count(vi.name))
            continue;
        for (int64_t d : vi.dims)
            if (d <= 0)
                fail("input " + vi.name + " has a symbolic shape");
        if (vi.dims.empty())
            fail("input " + vi.name + " has no shape");
        b.tensors[vi.name] = g->tensor(checkedDims(vi.dims, "input " + vi.name));
    }
    for (auto &nd : m.nodes) {
        const std::string &op = nd.op;
        if (op == "Constant" && !nd.outputs.empty()) {
            if (!nd.has("value") || nd.attrs.at("value").kind != Attr::Tensor)
                fail("Constant without a value tensor");
            b.consts[nd.outputs[0]] = nd.attrs.at("value").t;
            continue;
        }
        if (nd.outputs.empty() || nd.inputs.empty())
            fail("node " + nd.name + " (" + op + ") has no inputs or outputs");
        {
            // operands every form of the operator has
            static const std::map<std::string, size_t> kOperands = {
                {"Conv", 2}, {"Add", 2}, {"Mul", 2}, {"Sub", 2}, {"Div", 2}, {"MatMul", 2},
                {"Gemm", 2}, {"Gather", 2}, {"Reshape", 2}, {"Pow", 2}, {"Slice", 3},
                {"BatchNormalization", 5}, {"LayerNormalization", 2}};
            auto need = kOperands.find(op);
            if (need != kOperands.end() && nd.inputs.size() < need->second)
                fail(op + " with " + std::to_string(nd.inputs.size()) + " inputs");
        }
        if (op == "Shape") {
            Array a;
            for (int d : b.in(nd.inputs[0])->getDims())
                a.v.push_back(d);
            a.dims = {(int64_t)a.v.size()};
            a.integral = true;
            b.consts[nd.outputs[0]] = a;
            continue;
        }
        Tensor *x = b.in(nd.inputs[0]);
        const Dim xd = x->getDims();
        const int rank = (int)xd.size();
        Tensor *out = nullptr;
        auto axisOf = [&](int64_t a) { return (int)(((a % rank) + rank) % rank); };
        if (op == "Conv") {
            Tensor *w = b.in(nd.inputs[1]);
            Tensor *bias = nd.inputs.size() > 2 ? b.in(nd.inputs[2]) : nullptr;
            const int nsp = rank - 2;
            if (nd.gets("auto_pad", "NOTSET") != "NOTSET")
                fail("Conv: auto_pad is not supported");
            if (nsp != 2 && nsp != 3)
                fail("Conv with " + std::to_string(nsp) + " spatial dims");
            const std::vector<int> pads = symmetricPads(nd, nsp);
            const std::vector<int> st = intsOr(nd, "strides", nsp, 1);
            const std::vector<int> dil = intsOr(nd, "dilations", nsp, 1);
            const Dim wdims = w->getDims();
            const int64_t group = nd.geti("group", 1);
            if ((int)wdims.size() != rank || group < 1 || wdims[1] * group != xd[1] ||
                wdims[0] % group != 0)
                fail("Conv: filters " + std::to_string(wdims.size()) + "-d / group " +
                     std::to_string(group) + " do not fit the input");
            for (int i = 0; i < nsp; ++i)
                if (xd[2 + i] + 2 * pads[i] < dil[i] * (wdims[2 + i] - 1) + 1)
                    fail("Conv: the filter is larger than the padded input");
            if (bias && bias->size() != (size_t)wdims[0])
                fail("Conv: the bias is not one value per filter");
            if (nsp == 2) {
                out = resultOf(g->conv(x, w, pads[0], pads[1], st[0], st[1], dil[0], dil[1], bias));
            } else {
                const Dim wd = w->getDims();
                Dim od = {xd[0], wd[0]};
                for (int i = 0; i < 3; ++i)
                    od.push_back((xd[2 + i] + 2 * pads[i] - dil[i] * (wd[2 + i] - 1) - 1) / st[i] + 1);
                out = b.fresh(od);
                g->conv3d(x, w, out, Dim(pads.begin(), pads.end()), Dim(st.begin(), st.end()),
                          Dim(dil.begin(), dil.end()), bias);
            }
        } else if (op == "Relu" || op == "Sigmoid" || op == "Tanh" || op == "Gelu" ||
                   op == "Identity" || op == "Cast" || op == "Dropout") {
            if (op == "Gelu" && nd.gets("approximate", "none") != "none")
                fail("Gelu: the exact form only");
            out = b.fresh(xd);
            if (op == "Relu")
                g->relu(x, out);
            else if (op == "Sigmoid")
                g->sigmoid(x, out);
            else if (op == "Tanh")
                g->tanh(x, out);
            else if (op == "Gelu")
                g->gelu(x, out);
            else
                g->identity(x, out);
        } else if (op == "Add" || op == "Mul" || op == "Sub" || op == "Div") {
            Tensor *y = b.in(nd.inputs[1]);
            Tensor *big = x->size() >= y->size() ? x : y, *small = big == x ? y : x;
            const Dim bd = big->getDims();
            Dim sd = small->getDims();
            while (sd.size() > 1 && sd[0] == 1)
                sd.erase(sd.begin());
            const bool trailing =
                sd.size() <= bd.size() && std::equal(sd.begin(), sd.end(), bd.end() - sd.size());
            if (!trailing && small->size() != 1)
                fail(op + ": only trailing-dimension broadcast is supported");
            out = b.fresh(bd);
            if (op == "Add")
                g->add({x, y}, out);
            else if (op == "Mul")
                g->mul({x, y}, out);
            else if (op == "Sub")
                g->sub(x, y, out);
            else
                g->div(x, y, out);
        } else if (op == "MaxPool" || op == "AveragePool") {
            const std::vector<int64_t> k = nd.getis("kernel_shape");
            if (nd.geti("ceil_mode", 0) || k.size() != 2 || rank != 4)
                fail(op + ": ceil_mode / non-2-D pooling is not supported");
            const std::vector<int> pads = symmetricPads(nd, 2);
            const std::vector<int> st = intsOr(nd, "strides", 2, 1);
            // the backend's average leaves padding out of the divisor (ONNX's default and
            // the reference's cuDNN mode); max pooling is built without dilation
            if (op == "AveragePool" && nd.geti("count_include_pad", 0) && (pads[0] || pads[1]))
                fail("AveragePool: count_include_pad=1 with padding is not supported");
            for (int d : intsOr(nd, "dilations", 2, 1))
                if (d != 1)
                    fail(op + ": dilated pooling is not supported");
            Dim od = {xd[0], xd[1]};
            for (int i = 0; i < 2; ++i) {
                if (k[i] < 1 || k[i] > xd[2 + i] + 2 * pads[i])
                    fail(op + ": window of " + std::to_string(k[i]));
                od.push_back((xd[2 + i] + 2 * pads[i] - (int)k[i]) / st[i] + 1);
            }
            out = b.fresh(od);
            if (op == "MaxPool")
                g->maxpool(x, out, (int)k[0], (int)k[1], 1, 1, pads[0], pads[1], st[0], st[1]);
            else
                g->avgpool(x, out, (int)k[0], (int)k[1], pads[0], pads[1], st[0], st[1]);
        } else if (op == "GlobalAveragePool") {
            Dim od = {xd[0], xd[1]};
            od.resize(rank, 1);
            out = b.fresh(od);
            g->avgpool(x, out);
        } else if (op == "BatchNormalization") {
            if (nd.inputs.size() < 5)
                fail("BatchNormalization needs scale, bias, mean and variance");
            out = resultOf(g->batchnorm(x, b.in(nd.inputs[1]), b.in(nd.inputs[2]), b.in(nd.inputs[3]),
                                        b.in(nd.inputs[4]), (float)nd.getf("epsilon", 1e-5), 0.9f));
        } else if (op == "MatMul") {
            out = resultOf(g->matmul(x, b.in(nd.inputs[1])));
        } else if (op == "Gemm") {
            if (nd.getf("alpha", 1.0) != 1.0 || nd.getf("beta", 1.0) != 1.0)
                fail("Gemm with alpha / beta other than 1");
            Tensor *y = b.in(nd.inputs[1]);
            Tensor *bias = nd.inputs.size() > 2 ? b.in(nd.inputs[2]) : nullptr;
            const bool tb = nd.geti("transB", 0) != 0;
            const size_t nOut = tb ? y->getDims().front() : y->getDims().back();
            if (bias && bias->size() != nOut)
                fail("Gemm: C must be a vector of the output's last dim");
            out = resultOf(g->matmul(x, y, nd.geti("transA", 0) != 0, tb, bias));
        } else if (op == "Flatten") {
            const int64_t ax = nd.geti("axis", 1);
            if (ax < 0 || ax > rank)
                fail("Flatten: axis " + std::to_string(ax));
            int lead = 1, tail = 1;
            for (int i = 0; i < rank; ++i)
                (i < ax ? lead : tail) *= xd[i];
            out = b.fresh({lead, tail});
            g->flatten(x, out, (int)ax);
        } else if (op == "Reshape") {
            const Array &sh = b.constant(nd.inputs.at(1));
            Dim shape;
            long long known = 1;
            int hole = -1;
            for (size_t i = 0; i < sh.v.size(); ++i) {
                int v = (int)sh.v[i];
                if (v == 0) {
                    if (i >= xd.size())
                        fail("Reshape: 0 beyond the input's rank");
                    v = xd[i];
                }
                if (v == -1 && hole < 0)
                    hole = (int)i;
                else if (v < 1 || (known *= v) > (long long)x->size())
                    fail("Reshape: a shape that does not hold the input");
                shape.push_back(v);
            }
            if (hole >= 0)
                shape[hole] = (int)((long long)x->size() / std::max(known, 1ll));
            long long total = 1;
            for (int v : shape)
                total *= v;
            if (shape.empty() || total != (long long)x->size())
                fail("Reshape: a shape that does not hold the input");
            out = b.fresh(shape);
            g->reshape(x, out);
        } else if (op == "Transpose") {
            std::vector<int64_t> perm = nd.getis("perm");
            if (perm.empty())
                for (int i = rank - 1; i >= 0; --i)
                    perm.push_back(i);
            std::vector<PermItem> items;
            std::vector<bool> seen(rank, false);
            if ((int)perm.size() != rank)
                fail("Transpose: perm of another rank");
            for (int64_t p : perm) {
                if (p < 0 || p >= rank || seen[p])
                    fail("Transpose: perm is not a permutation");
                seen[p] = true;
                items.push_back(PermItem((int)p));
            }
            out = resultOf(g->transpose(x, -1, Perm(items), 2));
        } else if (op == "Concat") {
            TensorVec ins;
            const int ax = axisOf(nd.geti("axis", 0));
            for (auto &n : nd.inputs) {
                Tensor *t = b.in(n);
                Dim td = t->getDims();
                if ((int)td.size() != rank)
                    fail("Concat: inputs of different rank");
                for (int i = 0; i < rank; ++i)
                    if (i != ax && td[i] != xd[i])
                        fail("Concat: inputs that differ off the axis");
                ins.push_back(t);
            }
            out = resultOf(g->concat(ins, ax));
        } else if (op == "Split") {
            const int ax = axisOf(nd.geti("axis", 0));
            std::vector<int64_t> sizes = nd.getis("split");
            if (sizes.empty() && nd.inputs.size() > 1)
                for (double v : b.constant(nd.inputs[1]).v)
                    sizes.push_back((int64_t)v);
            if (sizes.empty())
                sizes.assign(nd.outputs.size(), xd[ax] / (int)nd.outputs.size());
            int64_t sum = 0;
            for (int64_t v : sizes)
                sum += v < 1 ? (int64_t)1 << 40 : v;
            if (sizes.size() != nd.outputs.size() || sum != xd[ax])
                fail("Split: sizes that do not add up to the axis");
            Operator *sp = g->split(x, ax, std::vector<int>(sizes.begin(), sizes.end()));
            if (!sp)
                fail("Split: the builder refused these sizes");
            const TensorVec &outs = sp->getOutputs();
            if (outs.size() != nd.outputs.size())
                fail("Split: " + std::to_string(nd.outputs.size()) + " outputs for " +
                     std::to_string(outs.size()) + " parts");
            for (size_t i = 0; i < outs.size(); ++i)
                b.tensors[nd.outputs[i]] = outs[i];
            continue;
        } else if (op == "Softmax") {
            if (axisOf(nd.geti("axis", -1)) != rank - 1)
                fail("Softmax over an axis other than the last");
            out = b.fresh(xd);
            g->softmax(x, out, rank - 1);
        } else if (op == "LayerNormalization") {
            if (axisOf(nd.geti("axis", -1)) != rank - 1 || nd.inputs.size() < 2)
                fail("LayerNormalization over more than the last axis");
            out = b.fresh(xd);
            g->layernorm(x, out, b.in(nd.inputs[1]),
                         nd.inputs.size() > 2 ? b.in(nd.inputs[2]) : nullptr,
                         (float)nd.getf("epsilon", 1e-5));
        } else if (op == "Gather") {
            out = resultOf(g->gather(x, b.in(nd.inputs.at(1)), axisOf(nd.geti("axis", 0))));
        } else if (op == "ReduceMean") {
            std::vector<int64_t> axes = nd.getis("axes");
            if (axes.empty() && nd.inputs.size() > 1)
                for (double v : b.constant(nd.inputs[1]).v)
                    axes.push_back((int64_t)v);
            if (axes.size() != 1 || !nd.geti("keepdims", 1))
                fail("ReduceMean over one axis with keepdims only");
            out = resultOf(g->reduceMean(x, axisOf(axes[0])));
        } else if (op == "Pad") {
            std::vector<int64_t> pads = nd.getis("pads");
            if (pads.empty() && nd.inputs.size() > 1)
                for (double v : b.constant(nd.inputs[1]).v)
                    pads.push_back((int64_t)v);
            if (nd.gets("mode", "constant") != "constant" || (int)pads.size() != 2 * rank)
                fail("Pad: constant mode with 2 * rank pads only");
            for (int64_t v : pads)
                if (v < 0 || v > (1 << 20))
                    fail("Pad: a pad of " + std::to_string(v));
            out = resultOf(g->pad(x, Dim(pads.begin(), pads.begin() + rank),
                                  Dim(pads.begin() + rank, pads.end())));
        } else if (op == "Slice") {
            // starts, ends, axes and steps as constants (opset 10 on); steps of 1 only
            auto listOf = [&](size_t i) {
                std::vector<double> v;
                if (nd.inputs.size() > i && !nd.inputs[i].empty())
                    v = b.constant(nd.inputs[i]).v;
                return v;
            };
            const std::vector<double> starts = listOf(1), ends = listOf(2), steps = listOf(4);
            std::vector<double> axes = listOf(3);
            if (axes.empty())
                for (size_t i = 0; i < starts.size(); ++i)
                    axes.push_back((double)i);
            if (starts.empty() || starts.size() != ends.size() || axes.size() != starts.size() ||
                (int)starts.size() > rank)
                fail("Slice: starts, ends and axes of different lengths");
            for (double st : steps)
                if (st != 1)
                    fail("Slice with a step other than 1");
            Dim begin(rank, 0), drop(rank, 0);
            std::vector<bool> seen(rank, false);
            for (size_t i = 0; i < axes.size(); ++i) {
                if (axes[i] != std::floor(axes[i]) || axes[i] < -rank || axes[i] >= rank)
                    fail("Slice: an axis out of range");
                const int ax = axisOf((int64_t)axes[i]);
                if (seen[ax])
                    fail("Slice: an axis named twice");
                seen[ax] = true;
                const double n = xd[ax];
                double lo = starts[i] < 0 ? starts[i] + n : starts[i];
                double hi = ends[i] < 0 ? ends[i] + n : ends[i];
                lo = std::min(std::max(lo, 0.0), n);
                hi = std::min(std::max(hi, 0.0), n);
                if (!(hi > lo))
                    fail("Slice: an empty range");
                begin[ax] = (int)lo;
                drop[ax] = (int)(n - hi);
            }
            out = resultOf(g->slice(x, begin, drop));
        } else if (op == "Pow") {
            const Array &e = b.constant(nd.inputs.at(1));
            const double p = e.v.empty() ? -1 : e.v[0];
            if (p != std::floor(p) || p < 0 || p > 64)
                fail("Pow with a non-integer exponent");
            out = resultOf(g->pow(x, (int)p));
        } else {
            fail("ONNX operator " + op + " is not supported");
        }
        if (!out)
            fail(op + ": the builder refused these shapes");
        b.tensors[nd.outputs[0]] = out;
    }
}

} // namespace

bool GraphBase::importOnnx(const char *net) {
    Graph *g = dynamic_cast<Graph *>(this);
    if (!g || !net) {
        std::fprintf(stderr, "[pet] importOnnx: needs a Graph and a file name\n");
        return false;
    }
    try {
        std::ifstream f(net, std::ios::binary);
        if (!f)
            fail("cannot open the file");
        std::vector<uint8_t> data((std::istreambuf_iterator<char>(f)),
                                  std::istreambuf_iterator<char>());
        Model m = parse(data);
        foldBatchnorm(m);
        InvalidOperandsThrow guard; // operands a builder rejects: a message, not an abort
        build(g, m);
    } catch (const std::exception &e) {
        std::fprintf(stderr, "[pet] importOnnx(%s): %s\n", net, e.what());
        return false;
    }
    updateConnection();
    return true;
}

} // namespace tpm
