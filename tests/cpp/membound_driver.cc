// MemBoundOp on the device against the reference's own evaluation: expressions are built
// with the reference's nnet tree (compiled unchanged), evaluated for every output position
// by nnet::Interpreter (src/nnet/Visitor/Interpreter.cc, what MemBoundOp::compute runs
// upstream, src/Graph/operator.cc:3601-3644), and by MemBoundOp::compute here, which
// flattens the tree and runs it on the GPU. Values are small integers, so the two must
// agree exactly. Also checks the CPU oracle's interpreter on the same flattened programs
// (it is linked into this binary only).
#include "graph.h"
#include "nnet/Visitor/Interpreter.h"
#include "nnet/expr.h"
#include "nnet/iterator_table.h"
#include "nnet/nmutator.h"
#include "operator.h"

#include <cstdio>
#include <cstdlib>
#include <map>

using namespace tpm;

extern "C" int oracle_expr_f32(const int *code, int ncode, const float *const *in, float *out);

static int failures = 0;

// withInterpreter: the reference's interpreter has no case for ReLU / tanh nodes
// (src/nnet/Visitor/Interpreter.cc has no visit_ for FuncNode); such expressions are
// checked against the oracle's interpreter alone.
static void check(const char *name, nnet::Expr expr, const std::vector<nnet::Tensor> &nnetIn,
                  bool withInterpreter = true) {
    auto range = nnet::as<nnet::RangeOpNode>(expr);
    Graph g;
    TensorVec ins;
    std::unordered_map<std::string, nnet::Ref<std::vector<int>>> data;
    unsigned state = 12345;
    for (auto &t : nnetIn) {
        Dim d(t->getShape().begin(), t->getShape().end());
        Tensor *ht = g.tensor(d);
        std::vector<float> v(ht->size());
        auto iv = nnet::make_ref<std::vector<int>>(ht->size());
        for (size_t i = 0; i < v.size(); ++i) {
            state = state * 1664525u + 1013904223u;
            int x = (int)((state >> 16) % 7u) - 3;
            v[i] = (float)x;
            (*iv)[i] = x;
        }
        ht->setData(v.data());
        ins.push_back(ht);
        data[t->getName()] = iv;
    }
    auto shape = range->getOutputShape();
    Tensor *out = g.tensor(Dim(shape.begin(), shape.end()));
    auto op = static_cast<MemBoundOp *>(g.membound(ins, {out}, nnetIn, expr, 0.01));
    if (op->program().empty()) {
        std::printf("[ FAIL ] %s: the expression does not flatten\n", name);
        ++failures;
        return;
    }
    if (op->compute() == nullptr) {
        std::printf("[ FAIL ] %s: did not run: %s\n", name, pet_hip_last_error());
        ++failures;
        return;
    }
    const float *got = out->getDataPtr();
    // the reference's interpreter, every output position
    // the oracle on the flattened program
    std::vector<const float *> ptrs;
    for (auto t : ins)
        ptrs.push_back(t->getDataPtr());
    std::vector<float> viaOracle(out->size());
    int orc = oracle_expr_f32(op->program().data(), (int)op->program().size(), ptrs.data(),
                              viaOracle.data());
    std::vector<int> want;
    if (withInterpreter)
        want = nnet::Interpreter(data).interpretAllOutput(range);
    else
        for (float v : viaOracle)
            want.push_back((int)v);
    size_t bad = 0, badOracle = 0;
    for (size_t i = 0; i < out->size(); ++i) {
        bad += got[i] != (float)want[i];
        badOracle += viaOracle[i] != (float)want[i];
    }
    if (want.size() != out->size() || bad || badOracle || orc) {
        std::printf("[ FAIL ] %s: %zu of %zu device values and %zu oracle values differ from "
                    "nnet::Interpreter\n", name, bad, out->size(), badOracle);
        ++failures;
    } else {
        std::printf("[  OK  ] %s: %zu values, %zu program words\n", name, out->size(),
                    op->program().size());
    }
}

// The reference's own conversion of an operator into a MemBound operator
    // (NMutator::runSingleOpToNaiveMembound, src/nnet/nmutator.cc:42-58): the
    // convolution and the MemBound operator that states it must agree on the device
static void naiveMemboundOfAConvolution() {
    Graph g;
    Tensor *x = g.tensor({2, 4, 6, 6}), *k = g.tensor({8, 4, 3, 3});
    g.conv(x, k, 1, 1);
    g.updateConnection();
    SubGraph in(g.getOperators());
    int seed = 5;
    for (auto t : in.getInputs())
        t->dataRand(seed++);
    NMutator mutator;
    mutator.setToNaiveMembound();
    std::vector<SubGraph *> outs;
    mutator.run(&in, outs);
    bool ok = outs.size() == 1 && outs[0]->getOperators().size() == 1 &&
              outs[0]->getOperators()[0]->getType() == Operator::MemBound;
    if (ok) {
        std::map<uint64_t, Tensor *> byHash;
        for (auto t : in.getInputs())
            byHash[t->getHash()] = t;
        for (auto t : outs[0]->getInputs())
            t->setData(byHash.at(t->getHash())->getDataPtr());
        ok = in.compute() && outs[0]->compute();
        const Tensor *a = in.getOutputs()[0], *b = outs[0]->getOutputs()[0];
        ok = ok && a->size() == b->size();
        for (size_t i = 0; ok && i < a->size(); ++i)
            ok = const_cast<Tensor *>(a)->getDataPtr()[i] ==
                 const_cast<Tensor *>(b)->getDataPtr()[i];
    }
    std::printf("[ %s ] NMutator naive MemBound of a convolution equals the convolution\n",
                ok ? " OK " : "FAIL");
    failures += !ok;
}

#define VAR(name) auto name = nnet::make_ref<nnet::VarNode>(#name)

int main() {
    using namespace nnet;
    {   // 3x3 convolution, padded reads: the reference's own pattern (iterator_table.cc:513-527)
        const int N = 2, C = 3, H = 6, W = 5, F = 4, R = 3, S = 3;
        auto A = makeTensor("A", {N, C, H, W}, {0, 0, 1, 1});
        auto K = makeTensor("K", {F, C, R, S});
        check("conv 3x3", ConvPattern::getExpr(A, K, N, C, H, W, F, R, S), {A, K});
    }
    {   // band products (iterator_table.cc:596-630)
        auto [e1, in1] = Sg2bmmPattern::getExpr(2, 12, 5, 3, 2);
        check("g2bmm", e1, {in1.first, in1.second});
        auto [e2, in2] = LongformerGBMMPattern::getExpr(2, 12, 3, 5, 2);
        check("gbmml", e2, {in2.first, in2.second});
        auto [e3, in3] = MatmulPattern::getExpr(false, false, 2, 5, 7, 6);
        check("matmul", e3, {in3.first, in3.second});
    }
    {   // a layout move with division and remainder, then a second stage reading the first in
        // its padding, with ReLU
        VAR(b); VAR(c); VAR(h); VAR(w);
        auto X = makeTensor("X", {1, 3, 8, 8});
        auto s2b = makeRangeOperator(
            {{b, {0, 4}}, {c, {0, 3}}, {h, {0, 4}}, {w, {0, 4}}}, {},
            makeSubscript(X, {make_ref<ConstantNode>(0), c, h * 2 + b / 2, w * 2 + b % 2}));
        check("space to batch", s2b, {X});
        VAR(i); VAR(p);
        auto V = makeTensor("V", {8});
        auto inner = makeRangeOperator({{p, {0, 8}}}, {}, makeSubscript(V, {p}) * 3, {2});
        auto outer = makeRangeOperator({{i, {0, 12}}}, {}, makeSubscript(inner, {i - 2}));
        check("nested range read in its padding", outer, {V});
        auto act = makeRangeOperator(
            {{i, {0, 8}}}, {}, make_ref<FuncNode>(makeSubscript(V, {i}), FuncType::Relu));
        check("ReLU node (oracle only)", act, {V}, false);
    }
    {   // transposed convolution as the search writes it (iterator_table.cc:544-594)
        const int N = 1, C = 2, H = 2, W = 2, F = 3, R = 4, S = 4;
        auto A = makeTensor("A", {N, H, W, F}, {0, R - 2, R - 2, 0});
        auto K = makeTensor("K", {R, S, F, C});
        check("conv transpose 4x4 / 2", ConvTransPattern::getExpr(A, K, N, C, H, W, F, R, S),
              {A, K});
    }
    naiveMemboundOfAConvolution();
    std::printf("%d failed\n", failures);
    std::fflush(stdout);
    std::_Exit(failures ? 1 : 0);
}
