#include <cmath>
#include "graph.h"
#include "perf_engine.h"

#include <algorithm>
#include <set>
#include <functional>
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
// NCHW -> NHWF, [f,c,r,s] -> [r,s,f,c] and NHWC -> NCHW around ConvTransOp
// (src/Graph/graph.cc:90-131).
Tensor *Graph::setConvTransInput(Tensor *input) {
    return own(new TransposeOp(input, -1, {0, 2, 3, 1}))->getOutputs()[0];
}
Tensor *Graph::setConvTransWeight(Tensor *weight) {
    weight->setType(Tensor::Weight);
    return own(new TransposeOp(weight, -1, {2, 3, 0, 1}))->getOutputs()[0];
}
Tensor *Graph::setConvTransOutput(Tensor *outputTrans, Tensor *output) {
    if (output == nullptr)
        return own(new TransposeOp(outputTrans, -1, {0, 3, 1, 2}))->getOutputs()[0];
    own(new TransposeOp(outputTrans, output, -1, {0, 3, 1, 2}));
    return output;
}
Operator *Graph::convTrans(Tensor *input, Tensor *weight, Tensor *output, int ph, int pw, int sh,
                           int sw, int dh, int dw, int oph, int opw, Tensor *bias) {
    input = setConvTransInput(input);
    weight = setConvTransWeight(weight);
    auto op = own(new ConvTransOp(input, weight, ph, pw, sh, sw, dh, dw, oph, opw, bias));
    setConvTransOutput(op->getOutputs()[0], output);
    return op;
}
Operator *Graph::convTrans(Tensor *input, Tensor *weight, Tensor *output,
                           ConvTransOp::PaddingMode pm, int sh, int sw, int dh, int dw, int oph,
                           int opw, Tensor *bias) {
    input = setConvTransInput(input);
    weight = setConvTransWeight(weight);
    auto op = own(new ConvTransOp(input, weight, pm, sh, sw, dh, dw, oph, opw, bias));
    setConvTransOutput(op->getOutputs()[0], output);
    return op;
}
Operator *Graph::g2bmm(Tensor *A, Tensor *B, Tensor *C, int width, int dilation, Tensor *bias) {
    return own(new G2BMMOp(A, B, C, width, dilation, bias));
}
Operator *Graph::g2bmm(Tensor *A, Tensor *B, int width, int dilation, Tensor *bias) {
    return own(new G2BMMOp(A, B, width, dilation, bias));
}
Operator *Graph::gbmml(Tensor *A, Tensor *B, Tensor *C, int dilation, Tensor *bias) {
    return own(new GBMMLOp(A, B, C, dilation, bias));
}
Operator *Graph::gbmml(Tensor *A, Tensor *B, int dilation, Tensor *bias) {
    return own(new GBMMLOp(A, B, dilation, bias));
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
Operator *Graph::div(Tensor *a, Tensor *b, Tensor *output) {
    return own(new DivOp({a, b}, output));
}
Operator *Graph::div(Tensor *a, Tensor *b) { return own(new DivOp({a, b})); }
Operator *Graph::pow(Tensor *input, Tensor *output, int pow) {
    return own(new PowOp(input, output, pow));
}
Operator *Graph::pow(Tensor *input, int pow) { return own(new PowOp(input, pow)); }
Operator *Graph::gather(Tensor *data, Tensor *indices, Tensor *output, int axis) {
    return own(new GatherOp(data, indices, output, axis));
}
Operator *Graph::gather(Tensor *data, Tensor *indices, int axis) {
    return own(new GatherOp(data, indices, axis));
}
Operator *Graph::reduceMean(Tensor *input, Tensor *output, int axis) {
    return own(new ReduceMeanOp(input, output, axis));
}
Operator *Graph::reduceMean(Tensor *input, int axis) {
    return own(new ReduceMeanOp(input, axis));
}
Operator *Graph::batchnorm(Tensor *input, Tensor *scale, Tensor *bias, Tensor *mean, Tensor *var,
                           Tensor *output, float epsilon, float momentum) {
    return own(new BatchNormOp(input, scale, bias, mean, var, output, epsilon, momentum));
}
Operator *Graph::batchnorm(Tensor *input, Tensor *scale, Tensor *bias, Tensor *mean, Tensor *var,
                           float epsilon, float momentum) {
    return own(new BatchNormOp(input, scale, bias, mean, var, epsilon, momentum));
}
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

namespace {
// While a graph is evaluated for comparison (compute, point compute, verification)
// split contractions add their partial sums in a fixed order, so that equal inputs
// give equal results from one evaluation to the next.
struct OrderedSums {
    int before = 0;
    OrderedSums() {
        pet_hip_get_deterministic(&before);
        pet_hip_set_deterministic(1);
    }
    ~OrderedSums() { pet_hip_set_deterministic(before); }
};
} // namespace

bool SubGraph::compute() {
    OrderedSums ordered;
    OpVec order;
    if (!topoOrder(order))
        return false;
    for (auto op : order)
        if (op->compute() == nullptr)
            return false;
    return petOk(pet_hip_stream_sync(petStream()), "pet_hip_stream_sync");
}

const std::pair<bool, VType> SubGraph::compute(const Dim &point, size_t outputId, bool) const {
    if (outputId >= outputs.size())
        return {false, 0};
    Tensor *out = outputs[outputId];
    if (!out->isComputed()) {
        OrderedSums ordered;
        OpVec order;
        if (!topoOrder(order))
            return {false, 0};
        for (auto op : order)
            if (op->compute() == nullptr) {
                if (hostTrace())
                    std::fprintf(stderr, "[pet] graph point compute: %s failed\n",
                                 op->toString().c_str());
                return {false, 0};
            }
        if (!petOk(pet_hip_stream_sync(petStream()), "pet_hip_stream_sync"))
            return {false, 0};
    }
    if (out->getOffset(point) == (size_t)-1) {
        if (hostTrace())
            std::fprintf(stderr, "[pet] graph point compute: point outside output %s\n",
                         dimToString(out->getDims()).c_str());
        return {false, 0};
    }
    VType value = out->getData(point);
    if (hostTrace())
        std::fprintf(stderr, "[pet] graph %p output %zu %s at %s = %g\n", (const void *)this,
                     outputId, dimToString(out->getDims()).c_str(), dimToString(point).c_str(),
                     (double)value);
    return {true, value};
}

void SubGraph::cleanConnection() {
    for (auto t : tensors) {
        t->setOutputOf(nullptr);
        t->setInputOf({});
    }
    for (auto op : ops) {
        op->setPredecessors({});
        op->setSuccessors({});
    }
    inputs.clear();
    outputs.clear();
}

int SubGraph::findTensor(Tensor *tensor, int ntensor) {
    int n = ntensor == 0 ? (int)tensors.size() : std::min(ntensor, (int)tensors.size());
    for (int i = 0; i < n; ++i)
        if (tensors[i] == tensor)
            return i;
    return -1;
}

bool SubGraph::resetOps(OpVec oplist, size_t ntensor) {
    ntensor = ntensor == 0 ? tensors.size() : std::min(ntensor, tensors.size());
    hash = 2147483647;
    // The operators of the previous list are borrowed and may be gone by now (the mutation
    // generator deletes its candidate operators at the start of every run,
    // src/Mutant/generator.cc:84-87, while its scratch graph still lists them): only the
    // graph's own tensors are reset here, and the operators of the new list below.
    for (auto t : tensors) {
        t->setOutputOf(nullptr);
        t->setInputOf({});
    }
    inputs.clear();
    outputs.clear();
    ops = std::move(oplist);
    for (auto op : ops) {
        op->setPredecessors({});
        op->setSuccessors({});
    }
    for (auto op : ops) {
        for (auto t : op->getInputs()) {
            if (findTensor(t) < 0)
                return false;
            t->addInputOf(op);
        }
        for (auto t : op->getOutputs()) {
            if (findTensor(t) < 0)
                return false;
            t->setOutputOf(op);
        }
    }
    for (size_t i = 0; i < ntensor; ++i) {
        Tensor *t = tensors[i];
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
    if (hostTrace()) {
        std::fprintf(stderr, "[pet] resetOps: %zu ops, %zu inputs, %zu outputs:", ops.size(),
                     inputs.size(), outputs.size());
        for (auto op : ops)
            std::fprintf(stderr, " %s;", op->toString().c_str());
        std::fprintf(stderr, "\n");
    }
    return true;
}

bool SubGraph::verification(SubGraph *mutant, bool) {
    if (inputs.size() != mutant->getInputs().size() || outputs.size() != mutant->getOutputs().size())
        return false;
    for (size_t i = 0; i < inputs.size(); ++i) {
        Tensor *a = inputs[i], *b = mutant->getInputs()[i];
        if (a->size() != b->size())
            return false;
        a->dataRand((int)i + 1);
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
        // The reference compares wrapping uint32 values, exact at any depth
        // (include/common.h:137). fp32 sums of dataRand's small integers are exact
        // up to 2^24, which one contraction stays under and two stacked ones need
        // not; beyond that the two graphs may round differently, so values that
        // large are compared to 2^-20 of their magnitude instead of bit for bit.
        for (size_t j = 0; j < a->size(); ++j)
            if (pa[j] != pb[j] &&
                !(std::fabs(pa[j]) >= 16777216.f &&
                  std::fabs(pa[j] - pb[j]) <= std::fabs(pa[j]) * 9.5367431640625e-7f)) {
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

// Wiring-aware hash (role of the reference's src/Graph/graph.cc:842-897): a
// node's value folds its operator hash with, per input, the tensor hash of a
// graph input or the value of the producing node; the graph's value folds the
// output tensors with their producers. Two graphs with the same operators but
// different connections hash differently, which the generator's visited-set
// pruning relies on.
uint64_t SubGraph::getHash() {
    if (hash != 2147483647)
        return hash;
    std::unordered_map<const Operator *, uint64_t> memo;
    std::function<uint64_t(Operator *)> nodeValue = [&](Operator *op) -> uint64_t {
        auto it = memo.find(op);
        if (it != memo.end())
            return it->second;
        memo[op] = 0; // a cycle would be a wiring bug; do not recurse forever
        uint64_t h = hashPack(op->getHash());
        for (auto t : op->getInputs()) {
            Operator *producer = t->getOutputOf();
            h = hashAppend(h, producer == nullptr ? t->getHash() : nodeValue(producer));
        }
        return memo[op] = hashPack(h);
    };
    uint64_t h = 0;
    for (auto t : outputs)
        if (t->getOutputOf() != nullptr)
            h = hashAppend(h, hashPack(hashAppend(t->getHash(), nodeValue(t->getOutputOf()))));
    hash = h;
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

namespace tpm {

uint64_t SubGraph::getCacheIdx(int level) {
    static const uint64_t factors[8] = {10000019, 10000079, 10000103, 10000121,
                                        10000139, 10000141, 10000169, 10000189};
    uint64_t h = 0;
    for (auto op : ops) {
        h = hashAppend(h, std::hash<uint64_t>()(op->getType()));
        if (level != 1)
            continue;
        size_t l = 0;
        for (auto in : op->getInputs()) {
            uint64_t th = 0;
            for (int d : in->getDims())
                th = hashAppend(th, (uint64_t)d * factors[l++ % 8]);
            h = hashAppend(h, th);
        }
    }
    return h;
}

int SubGraph::printBrief() {
    std::cout << "Subgraph[" << getHash() << "] brief\n    op num: " << ops.size()
              << "\n    input: ";
    for (auto t : inputs)
        std::cout << t->getHash() << " ";
    std::cout << "\n    output: ";
    for (auto t : outputs)
        if (t->isNotCounted())
            std::cout << "(" << t->getHash() << ") ";
        else
            std::cout << t->getHash() << " ";
    std::cout << std::endl;
    return 0;
}

int SubGraph::reset(std::vector<Tensor *> &input, std::vector<Tensor *> &output) {
    for (auto t : tensors)
        t->refresh();
    if (inputs.size() != input.size() || outputs.size() != output.size())
        return 1;
    for (size_t i = 0; i < input.size(); ++i)
        inputs[i]->replace(*input[i]);
    for (size_t i = 0; i < output.size(); ++i)
        outputs[i]->replace(*output[i]);
    return 0;
}

int SubGraph::split(std::shared_ptr<SubGraph> &master, std::shared_ptr<SubGraph> &slave,
                    std::vector<Operator *> &slaveOps) {
    std::set<Operator *> mine(ops.begin(), ops.end()), taken;
    for (auto op : slaveOps) {
        if (!mine.count(op)) {
            std::cout << "ERROR: [SubGraph::split] slave op not in subgraph." << std::endl;
            return 1;
        }
        taken.insert(op);
    }
    OpVec rest;
    for (auto op : ops)
        if (!taken.count(op))
            rest.push_back(op);
    master = std::make_shared<SubGraph>(rest);
    slave = std::make_shared<SubGraph>(slaveOps);
    return 0;
}

int SubGraph::merge(std::shared_ptr<SubGraph> &master, std::shared_ptr<SubGraph> &slave) {
    std::unordered_map<uint64_t, Tensor *> byHash;
    for (auto t : tensors)
        byHash.emplace(t->getHash(), t);
    OpVec all(ops.begin(), ops.end());
    auto mine = [&](Tensor *t) {
        auto it = byHash.find(t->getHash());
        return it == byHash.end() ? t : it->second;
    };
    for (auto op : slave->getOperators()) {
        TensorVec ins, outs;
        for (auto t : op->getInputs())
            ins.push_back(mine(t));
        for (auto t : op->getOutputs())
            outs.push_back(mine(t));
        op->setInputs(ins);
        op->setOutputs(outs);
        all.push_back(op);
    }
    master = std::make_shared<SubGraph>(all);
    return 0;
}

} // namespace tpm
