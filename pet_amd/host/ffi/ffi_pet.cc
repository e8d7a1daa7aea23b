// Python surface of the host layer: the module the reference builds from
// src/ffi/ffi_pet.cc:19-208 (cpp_module: Graph with its builder methods, SubGraph,
// CodeEngine, PerfEngine), so that python/cpp_plugin-style front ends can drive this
// backend. Same class and method names and argument orders; SearchEngine is absent
// (the reference's needs its nnet sources). Additions a GPU-side caller needs: tensor
// data in and out as numpy arrays, SubGraph.compute / perf, CodeEngine.instantiate.
#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include "code_engine.h"
#include "graph.h"
#include "operator.h"
#include "perf_engine.h"
#include "tensor.h"

namespace py = pybind11;
using namespace py::literals;
using namespace tpm;

namespace {

constexpr auto kRef = py::return_value_policy::reference_internal;

// "after" as Python writes it: a list whose items are ints or lists of ints
Perm permFrom(const py::list &after) {
    std::vector<PermItem> items;
    for (auto h : after) {
        if (py::isinstance<py::int_>(h))
            items.emplace_back(std::vector<int>{h.cast<int>()});
        else
            items.emplace_back(h.cast<std::vector<int>>());
    }
    return Perm(items);
}

py::array_t<float> tensorData(Tensor &t) {
    const float *p = t.getDataPtr();
    if (p == nullptr)
        throw std::runtime_error("tensor has no data");
    std::vector<py::ssize_t> shape(t.getDims().begin(), t.getDims().end());
    py::array_t<float> out(shape);
    std::memcpy(out.mutable_data(), p, t.size() * sizeof(float));
    return out;
}

void setTensorData(Tensor &t, py::array_t<float, py::array::c_style | py::array::forcecast> a) {
    if ((size_t)a.size() != t.size())
        throw std::runtime_error("array has " + std::to_string(a.size()) + " elements, tensor " +
                                 std::to_string(t.size()));
    if (!t.setData(a.data()))
        throw std::runtime_error("setData failed");
}

} // namespace

PYBIND11_MODULE(cpp_module, m) {
    m.doc() = "PET host layer on the MI355X backend";
    // From Python, operands a constructor rejects are a ValueError (pybind11 translates
    // std::invalid_argument), not the assertion that ends a C++ program: in force on the
    // importing thread for as long as the module lives.
    static InvalidOperandsThrow *operandErrors = new InvalidOperandsThrow();
    (void)operandErrors;

    py::class_<Tensor>(m, "Tensor")
        .def("getDims", [](const Tensor &t) { return t.getDims(); })
        .def("size", &Tensor::size)
        .def("getHash", &Tensor::getHash)
        .def("dataRand", [](Tensor &t, int seed) { return t.dataRand(seed); }, "seed"_a = 0)
        .def("setWeight", [](Tensor &t) { t.setType(Tensor::Weight); })
        .def("isWeight", [](const Tensor &t) { return t.getType() == Tensor::Weight; })
        .def("setData", &setTensorData)
        .def("getData", &tensorData);

    py::class_<Operator>(m, "Operator")
        .def("toString", &Operator::toString)
        .def("getInputs", [](Operator &op) { return op.getInputs(); }, kRef)
        .def("getOutputs", [](Operator &op) { return op.getOutputs(); }, kRef)
        .def("getOutput", [](Operator &op) { return op.getOutputs().at(0); }, kRef)
        .def("perf", [](Operator &op, std::shared_ptr<PerfEngine> pe) { return op.perf(pe.get()); })
        .def("setAct", [](Operator &op, int act) {
            if (auto c = dynamic_cast<ConvOp *>(&op))
                c->setAct((Operator::ActType)act);
            else if (auto c3 = dynamic_cast<Conv3dOp *>(&op))
                c3->setAct((Operator::ActType)act);
            else if (auto mm = dynamic_cast<MatmulOp *>(&op))
                mm->setAct((Operator::ActType)act);
            else
                throw std::runtime_error("operator has no fused activation");
        });

    py::class_<PermItem>(m, "PermItem")
        .def(py::init<>())
        .def(py::init<const std::vector<int> &>());
    py::class_<Perm>(m, "Perm")
        .def(py::init<const std::vector<PermItem> &>())
        .def(py::init(&permFrom));

    py::class_<Graph>(m, "Graph")
        .def(py::init<>())
        .def("tensor", py::overload_cast<const Dim &, const std::string &>(&Graph::tensor),
             "dims"_a, "dtype"_a = "FLOAT", kRef)
        .def("conv",
             py::overload_cast<Tensor *, Tensor *, Tensor *, int, int, int, int, int, int, Tensor *>(
                 &Graph::conv),
             "input"_a, "weight"_a, "output"_a, "ph"_a, "pw"_a, "sh"_a = 1, "sw"_a = 1,
             "dh"_a = 1, "dw"_a = 1, "bias"_a = nullptr, kRef)
        .def("conv3d", &Graph::conv3d, "input"_a, "weight"_a, "output"_a, "pad"_a, "stride"_a,
             "dilation"_a, "bias"_a = nullptr, kRef)
        .def("matmul",
             py::overload_cast<Tensor *, Tensor *, Tensor *, bool, bool, Tensor *>(&Graph::matmul),
             "A"_a, "B"_a, "C"_a, "transA"_a = false, "transB"_a = false, "bias"_a = nullptr, kRef)
        .def("convTrans",
             py::overload_cast<Tensor *, Tensor *, Tensor *, int, int, int, int, int, int, int, int,
                               Tensor *>(&Graph::convTrans),
             "input"_a, "weight"_a, "output"_a, "ph"_a, "pw"_a, "sh"_a = 1, "sw"_a = 1,
             "dh"_a = 1, "dw"_a = 1, "oph"_a = 0, "opw"_a = 0, "bias"_a = nullptr, kRef)
        .def("g2bmm",
             py::overload_cast<Tensor *, Tensor *, Tensor *, int, int, Tensor *>(&Graph::g2bmm),
             "A"_a, "B"_a, "C"_a, "width"_a, "dilation"_a, "bias"_a = nullptr, kRef)
        .def("gbmml",
             py::overload_cast<Tensor *, Tensor *, Tensor *, int, Tensor *>(&Graph::gbmml), "A"_a,
             "B"_a, "C"_a, "dilation"_a, "bias"_a = nullptr, kRef)
        .def("pad",
             py::overload_cast<Tensor *, Tensor *, const Dim &, const Dim &>(&Graph::pad), kRef)
        .def("slice",
             py::overload_cast<Tensor *, Tensor *, const Dim &, const Dim &>(&Graph::slice), kRef)
        .def("concat", py::overload_cast<const TensorVec &, Tensor *, int>(&Graph::concat), kRef)
        .def("split", py::overload_cast<Tensor *, const TensorVec &, int, int>(&Graph::split),
             kRef)
        .def("split",
             py::overload_cast<Tensor *, const TensorVec &, int, std::vector<int>>(&Graph::split),
             kRef)
        .def("transpose",
             py::overload_cast<Tensor *, Tensor *, int, const Perm &, int>(&Graph::transpose),
             "input"_a, "output"_a, "split"_a, "after"_a, "factor"_a = 2, kRef)
        .def("transpose",
             [](Graph &g, Tensor *in, Tensor *out, int split, const py::list &after, int factor) {
                 return g.transpose(in, out, split, permFrom(after), factor);
             },
             "input"_a, "output"_a, "split"_a, "after"_a, "factor"_a = 2, kRef)
        .def("flatten", &Graph::flatten, kRef)
        .def("extend", py::overload_cast<Tensor *, Tensor *, int, int>(&Graph::extend), kRef)
        .def("maxpool", &Graph::maxpool, kRef)
        .def("avgpool",
             py::overload_cast<Tensor *, Tensor *, int, int, int, int, int, int>(&Graph::avgpool),
             kRef)
        .def("avgpool", py::overload_cast<Tensor *, Tensor *>(&Graph::avgpool), kRef)
        .def("add", py::overload_cast<const TensorVec &, Tensor *>(&Graph::add), kRef)
        .def("sub", &Graph::sub, kRef)
        .def("mul", py::overload_cast<const TensorVec &, Tensor *>(&Graph::mul), kRef)
        .def("div", py::overload_cast<Tensor *, Tensor *, Tensor *>(&Graph::div), kRef)
        .def("pow", py::overload_cast<Tensor *, Tensor *, int>(&Graph::pow), kRef)
        .def("gather", py::overload_cast<Tensor *, Tensor *, Tensor *, int>(&Graph::gather), kRef)
        .def("reduceMean", py::overload_cast<Tensor *, Tensor *, int>(&Graph::reduceMean), kRef)
        .def("softmax", &Graph::softmax, kRef)
        .def("layernorm", &Graph::layernorm, "input"_a, "output"_a, "gamma"_a, "beta"_a,
             "eps"_a = 1e-5f, kRef)
        .def("reshape", &Graph::reshape, kRef)
        .def("identity", &Graph::identity, kRef)
        .def("relu", py::overload_cast<Tensor *, Tensor *>(&Graph::relu), kRef)
        .def("sigmoid", &Graph::sigmoid, kRef)
        .def("tanh", &Graph::tanh, kRef)
        .def("gelu", &Graph::gelu, kRef)
        .def("batchnorm",
             py::overload_cast<Tensor *, Tensor *, Tensor *, Tensor *, Tensor *, Tensor *, float,
                               float>(&Graph::batchnorm),
             "input"_a, "scale"_a, "bias"_a, "mean"_a, "var"_a, "output"_a, "epsilon"_a = 1e-5f,
             "momentum"_a = 0.9f, kRef)
        // the same builders making their own output tensor (the reference's C++ overloads)
        .def("conv",
             py::overload_cast<Tensor *, Tensor *, int, int, int, int, int, int, Tensor *>(
                 &Graph::conv),
             "input"_a, "weight"_a, "ph"_a, "pw"_a, "sh"_a = 1, "sw"_a = 1, "dh"_a = 1, "dw"_a = 1,
             "bias"_a = nullptr, kRef)
        .def("matmul", py::overload_cast<Tensor *, Tensor *, bool, bool, Tensor *>(&Graph::matmul),
             "A"_a, "B"_a, "transA"_a = false, "transB"_a = false, "bias"_a = nullptr, kRef)
        .def("pad", py::overload_cast<Tensor *, const Dim &, const Dim &>(&Graph::pad), kRef)
        .def("slice", py::overload_cast<Tensor *, const Dim &, const Dim &>(&Graph::slice), kRef)
        .def("concat", py::overload_cast<const TensorVec &, int>(&Graph::concat), kRef)
        .def("split", py::overload_cast<Tensor *, int, std::vector<int>>(&Graph::split), kRef)
        .def("transpose",
             [](Graph &g, Tensor *in, int split, const py::list &after, int factor) {
                 return g.transpose(in, split, permFrom(after), factor);
             },
             "input"_a, "split"_a, "after"_a, "factor"_a = 2, kRef)
        .def("add", py::overload_cast<const TensorVec &>(&Graph::add), kRef)
        .def("mul", py::overload_cast<const TensorVec &>(&Graph::mul), kRef)
        .def("div", py::overload_cast<Tensor *, Tensor *>(&Graph::div), kRef)
        .def("pow", py::overload_cast<Tensor *, int>(&Graph::pow), kRef)
        .def("gather", py::overload_cast<Tensor *, Tensor *, int>(&Graph::gather), kRef)
        .def("reduceMean", py::overload_cast<Tensor *, int>(&Graph::reduceMean), kRef)
        .def("relu", py::overload_cast<Tensor *>(&Graph::relu), kRef)
        .def("batchnorm",
             py::overload_cast<Tensor *, Tensor *, Tensor *, Tensor *, Tensor *, float, float>(
                 &Graph::batchnorm),
             "input"_a, "scale"_a, "bias"_a, "mean"_a, "var"_a, "epsilon"_a = 1e-5f,
             "momentum"_a = 0.9f, kRef)
        .def("setInputs", &Graph::setInputs)
        .def("setOutputs", &Graph::setOutputs)
        .def("getOperators", [](Graph &g) { return g.getOperators(); }, kRef)
        .def("getTensors", [](Graph &g) { return g.getTensors(); }, kRef)
        .def("updateConnection", &Graph::updateConnection)
        .def("importOnnx", [](Graph &g, const std::string &path) { return g.importOnnx(path.c_str()); })
        .def("exportOnnx", [](Graph &g, const std::string &path) { return g.exportOnnx(path.c_str()); });

    // dynamic attributes: Python code parks the Graph a SubGraph was cut from on it (the
    // SubGraph's operators keep pointing at that Graph's bias-like side tensors)
    py::class_<SubGraph, std::shared_ptr<SubGraph>>(m, "SubGraph", py::dynamic_attr())
        .def(py::init<>())
        .def(py::init<OpVec>())
        .def("getInputs", [](SubGraph &g) { return g.getInputs(); }, kRef)
        .def("getOutputs", [](SubGraph &g) { return g.getOutputs(); }, kRef)
        .def("getOperators", [](SubGraph &g) { return g.getOperators(); }, kRef)
        .def("compute", py::overload_cast<>(&SubGraph::compute))
        .def("exportOnnx",
             [](SubGraph &g, const std::string &path) { return g.exportOnnx(path.c_str()); })
        .def("verification", &SubGraph::verification, "mutant"_a, "isFullComputing"_a = true)
        .def("perf",
             [](SubGraph &g, std::shared_ptr<PerfEngine> pe, bool withPenalty) {
                 return g.perf(pe.get(), withPenalty);
             },
             "perfEngine"_a, "withPenalty"_a = true);

    py::class_<PerfEngine, std::shared_ptr<PerfEngine>>(m, "PerfEngine").def(py::init<>());

    py::class_<GraphExec>(m, "GraphExec")
        .def("launch", &GraphExec::launch)
        .def("sync", &GraphExec::sync)
        .def("time", &GraphExec::time, "warmup"_a = 100, "rounds"_a = 1000)
        .def("numKernelOps", &GraphExec::numKernelOps)
        .def("numAliasedOps", &GraphExec::numAliasedOps)
        .def("numFoldedOps", &GraphExec::numFoldedOps)
        .def("numHoistedFills", &GraphExec::numHoistedFills);

    py::class_<CodeEngine>(m, "CodeEngine")
        .def(py::init<>())
        .def("importPerfEngine", &CodeEngine::importPerfEngine)
        .def("genCode",
             py::overload_cast<std::shared_ptr<SubGraph> &, const std::string &>(
                 &CodeEngine::genCode))
        .def("genCode", py::overload_cast<std::shared_ptr<SubGraph> &>(&CodeEngine::genCode))
        .def("instantiate", [](CodeEngine &ce, std::shared_ptr<SubGraph> g) {
            auto exec = ce.instantiate(g);
            if (!exec)
                throw std::runtime_error("the graph could not be instantiated");
            return exec;
        });
}
