#include "graph.h"
#include "perf_engine.h"

#include <algorithm>
#include <unordered_map>

namespace tpm {

GraphBase::~GraphBase() {
    for (auto op : ops)
        delete op;
    for (auto t : tensors)
        delete t;
}

Tensor *GraphBase::tensor(const Dim &dims, Tensor::DataType dtype) {
    tensors.push_back(new Tensor(dims, Tensor::Input, dtype));
    return tensors.back();
}

Tensor *GraphBase::tensor(const Dim &dims, const std::string &dtype) {
    return tensor(dims, dtype == "INT32" || dtype == "Int32" ? Tensor::Int32 : Tensor::Float32);
}

void GraphBase::updateConnection() {
    for (auto t : tensors) {
        t->setInputOf({});
        t->setOutputOf(nullptr);
    }
    for (auto op : ops) {
        op->setPredecessors({});
        op->setSuccessors({});
    }
    for (auto op : ops) {
        for (auto t : op->getInputs())
            t->addInputOf(op);
        for (auto t : op->getOutputs())
            t->setOutputOf(op);
    }
    inputs.clear();
    outputs.clear();
    for (auto t : tensors) {
        Operator *producer = t->getOutputOf();
        for (auto consumer : t->getInputOf())
            if (producer != nullptr) {
                consumer->addPredecessors(producer);
                producer->addSuccessors(consumer);
            }
        if (!t->getInputOf().empty() && producer == nullptr)
            inputs.push_back(t);
        if (t->getInputOf().empty() && producer != nullptr)
            outputs.push_back(t);
    }
}

void GraphBase::removeOps(OpVec &removed) {
    for (auto op : removed) {
        auto it = std::find(ops.begin(), ops.end(), op);
        if (it != ops.end()) {
            ops.erase(it);
            delete op;
        }
    }
    updateConnection();
}

bool GraphBase::topoOrder(OpVec &order) const {
    std::unordered_map<const Operator *, int> pending;
    OpVec ready;
    for (auto op : ops) {
        // count distinct pending producers through tensors (an op may consume
        // two outputs of the same producer)
        int n = (int)op->getPredecessors().size();
        pending[op] = n;
        if (n == 0)
            ready.push_back(op);
    }
    order.clear();
    for (size_t head = 0; head < ready.size(); ++head) {
        Operator *op = ready[head];
        order.push_back(op);
        for (auto suc : op->getSuccessors())
            if (--pending[suc] == 0)
                ready.push_back(suc);
    }
    return order.size() == ops.size();
}

// ---- Graph builders -------------------------------------------------------------

Operator *Graph::own(Operator *op) {
    ops.push_back(op);
    // tensors the operator created for itself join the graph's ownership
    for (auto t : op->getOutputs())
        if (std::find(tensors.begin(), tensors.end(), t) == tensors.end())
            tensors.push_back(t);
    return op;
}

Operator *Graph::conv(Tensor *input, Tensor *weight, Tensor *output, int ph, int pw, int sh,
                      int sw, int dh, int dw, Tensor *bias) {
    return own(new ConvOp(input, weight, output, ph, pw, sh, sw, dh, dw, bias));
}
Operator *Graph::conv(Tensor *input, Tensor *weight, int ph, int pw, int sh, int sw, int dh,
                      int dw, Tensor *bias) {
    return own(new ConvOp(input, weight, ph, pw, sh, sw, dh, dw, bias));
}
Operator *Graph::conv(Tensor *input, Tensor *weight, Tensor *output, ConvOp::PaddingMode pm,
                      int sh, int sw, int dh, int dw, Tensor *bias) {
    return own(new ConvOp(input, weight, output, pm, sh, sw, dh, dw, bias));
}
Operator *Graph::conv(Tensor *input, Tensor *weight, ConvOp::PaddingMode pm, int sh, int sw,
                      int dh, int dw, Tensor *bias) {
    return own(new ConvOp(input, weight, pm, sh, sw, dh, dw, bias));
}
Operator *Graph::conv3d(Tensor *input, Tensor *weight, Tensor *output, const Dim &pad,
                        const Dim &stride, const Dim &dilation, Tensor *bias) {
    return own(new Conv3dOp(input, weight, output, pad, stride, dilation, bias));
}
Operator *Graph::matmul(Tensor *A, Tensor *B, Tensor *C, bool transA, bool transB, Tensor *bias) {
    return own(new MatmulOp(A, B, C, transA, transB, bias));
}
Operator *Graph::matmul(Tensor *A, Tensor *B, bool transA, bool transB, Tensor *bias) {
    return own(new MatmulOp(A, B, transA, transB, bias));
}
Operator *Graph::pad(Tensor *input, Tensor *output, const Dim &begin, const Dim &end) {
    return own(new PadOp(input, output, begin, end));
}
Operator *Graph::pad(Tensor *input, const Dim &begin, const Dim &end) {
    return own(new PadOp(input, begin, end));
}
Operator *Graph::slice(Tensor *input, Tensor *output, const Dim &begin, const Dim &end) {
    return own(new SliceOp(input, output, begin, end));
}
Operator *Graph::slice(Tensor *input, const Dim &begin, const Dim &end) {
    return own(new SliceOp(input, begin, end));
}
Operator *Graph::concat(const TensorVec &ins, Tensor *output, int dim) {
    return own(new ConcatOp(ins, output, dim));
}
Operator *Graph::concat(const TensorVec &ins, int dim) { return own(new ConcatOp(ins, dim)); }
Operator *Graph::split(Tensor *input, const TensorVec &outs, int dim, int num) {
    return own(new SplitOp(input, outs, dim, std::vector<int>(num, 1)));
}
Operator *Graph::split(Tensor *input, int dim, int num) {
    return own(new SplitOp(input, dim, num));
}
Operator *Graph::split(Tensor *input, const TensorVec &outs, int dim, std::vector<int> sizes) {
    return own(new SplitOp(input, outs, dim, sizes));
}
Operator *Graph::split(Tensor *input, int dim, std::vector<int> sizes) {
    return own(new SplitOp(input, dim, sizes));
}
Operator *Graph::transpose(Tensor *input, Tensor *output, int split, const Perm &after,
                           int factor) {
    return own(new TransposeOp(input, output, split, after, factor));
}
Operator *Graph::transpose(Tensor *input, int split, const Perm &after, int factor) {
    return own(new TransposeOp(input, split, after, factor));
}
// "flatten" is a reshape to [prod(dims[:axis]), prod(dims[axis:])]
Operator *Graph::flatten(Tensor *input, Tensor *output, int axis) {
    const Dim &d = input->getDims();
    int a = 1, b = 1;
    for (int i = 0; i < (int)d.size(); ++i)
        (i < axis ? a : b) *= d[i];
    output->setDims({a, b});
    return own(new ReshapeOp(input, output));
}
Operator *Graph::extend(Tensor *input, Tensor *output, int dim, int num) {
    return own(new ExtendOp(input, output, dim, num));
}
Operator *Graph::extend(Tensor *input, int dim, int num) {
    return own(new ExtendOp(input, dim, num));
}
Operator *Graph::maxpool(Tensor *input, Tensor *output, int kh, int kw, int dh, int dw, int ph,
                         int pw, int sh, int sw) {
    return own(new MaxPoolOp(input, output, kh, kw, dh, dw, ph, pw, sh, sw));
}
Operator *Graph::avgpool(Tensor *input, Tensor *output, int kh, int kw, int ph, int pw, int sh,
                         int sw) {
    return own(new AvgPoolOp(input, output, kh, kw, ph, pw, sh, sw));
}
Operator *Graph::avgpool(Tensor *input, Tensor *output) {
    return own(new AvgPoolOp(input, output));
}
Operator *Graph::add(const TensorVec &ins, Tensor *output) { return own(new AddOp(ins, output)); }
Operator *Graph::add(const TensorVec &ins) { return own(new AddOp(ins)); }
Operator *Graph::sub(Tensor *a, Tensor *b, Tensor *output) { return own(new SubOp(a, b, output)); }
Operator *Graph::mul(const TensorVec &ins, Tensor *output) { return own(new MulOp(ins, output)); }
Operator *Graph::mul(const TensorVec &ins) { return own(new MulOp(ins)); }
Operator *Graph::reshape(Tensor *input, Tensor *output) {
    return own(new ReshapeOp(input, output));
}
Operator *Graph::identity(Tensor *input, Tensor *output) {
    auto op = new IdentityOp(input, output);
    op->computeShape();
    return own(op);
}
Operator *Graph::relu(Tensor *input, Tensor *output) {
    return own(new ActivationOp(input, output, Operator::Relu));
}
Operator *Graph::relu(Tensor *input) { return own(new ActivationOp(input, Operator::Relu)); }
Operator *Graph::sigmoid(Tensor *input, Tensor *output) {
    return own(new ActivationOp(input, output, Operator::Sigmoid));
}
Operator *Graph::tanh(Tensor *input, Tensor *output) {
    return own(new ActivationOp(input, output, Operator::Tanh));
}
Operator *Graph::gelu(Tensor *input, Tensor *output) {
    return own(new ActivationOp(input, output, Operator::Gelu));
}
Operator *Graph::softmax(Tensor *input, Tensor *output, int axis) {
    return own(new SoftmaxOp(input, output, axis));
}
Operator *Graph::layernorm(Tensor *input, Tensor *output, Tensor *gamma, Tensor *beta, float eps) {
    return own(new LayerNormOp(input, output, gamma, beta, eps));
}

// ---- SubGraph ---------------------------------------------------------------------

SubGraph::SubGraph(OpVec oplist) {
    std::map<uint64_t, Tensor *> byHash;
    auto mirror = [&](Tensor *orig) {
        auto it = byHash.find(orig->getHash());
        if (it != byHash.end())
            return it->second;
        Tensor *t = orig->clone();
        tensors.push_back(t);
        byHash.emplace(orig->getHash(), t);
        return t;
    };
    for (auto orig : oplist) {
        Operator *op = orig->clone();
        ops.push_back(op);
        for (auto t : orig->getInputs())
            op->addInput(mirror(t));
        for (auto t : orig->getOutputs())
            op->addOutput(mirror(t));
    }
    updateConnection();
}

void SubGraph::resetComputed() {
    for (auto t : tensors)
        if (t->getOutputOf() != nullptr)
            t->setNotComputed();
}

bool SubGraph::compute() {
    OpVec order;
    if (!topoOrder(order))
        return false;
    for (auto op : order)
        if (op->compute() == nullptr)
            return false;
    return petOk(pet_hip_stream_sync(petStream()), "pet_hip_stream_sync");
}

const std::pair<bool, VType> SubGraph::compute(const Dim &point, size_t outputId, bool) {
    if (outputId >= outputs.size())
        return {false, 0};
    Tensor *out = outputs[outputId];
    if (!out->isComputed() && !compute())
        return {false, 0};
    if (out->getOffset(point) == (size_t)-1)
        return {false, 0};
    return {true, out->getData(point)};
}

bool SubGraph::verification(SubGraph *mutant, bool) {
    if (inputs.size() != mutant->getInputs().size() || outputs.size() != mutant->getOutputs().size())
        return false;
    for (size_t i = 0; i < inputs.size(); ++i) {
        Tensor *a = inputs[i], *b = mutant->getInputs()[i];
        if (a->size() != b->size())
            return false;
        a->dataRand((int)i);
        b->setData(a->getDataPtr());
    }
    resetComputed();
    mutant->resetComputed();
    if (!compute() || !mutant->compute())
        return false;
    for (size_t i = 0; i < outputs.size(); ++i) {
        Tensor *a = outputs[i], *b = mutant->getOutputs()[i];
        if (a->size() != b->size())
            return false;
        const VType *pa = a->getDataPtr(), *pb = b->getDataPtr();
        for (size_t j = 0; j < a->size(); ++j)
            if (pa[j] != pb[j]) {
                std::printf("[Wrong] output %zu element %zu: graph = %g mutant = %g\n", i, j,
                            (double)pa[j], (double)pb[j]);
                return false;
            }
    }
    return true;
}

double SubGraph::perf(PerfEngine *pe, bool withPenalty) {
    pe->setPenalty(withPenalty ? 1 : 0);
    double total = 0.0;
    for (auto op : ops)
        total += op->perf(pe, 200, 200);
    return total;
}

uint64_t SubGraph::getHash() {
    if (hash != 2147483647)
        return hash;
    uint64_t h = 0;
    OpVec order;
    topoOrder(order);
    for (auto op : order)
        h = hashAppend(h, op->getHash());
    hash = hashPack(h);
    return hash;
}

int SubGraph::print() {
    for (auto op : ops)
        op->print();
    return 0;
}

int SubGraph::getComputeOps(OpVec &out) {
    for (auto op : ops)
        if (op->isComputeOp())
            out.push_back(op);
    return (int)out.size();
}

} // namespace tpm
