// Graph containers (role of the reference's include/graph.h): the builder API
// the ONNX importer and the mutators call, connection inference, topological
// execution on the device and the original-vs-mutant check.
#pragma once
#include "common.h"
#include "operator.h"
#include "tensor.h"
#include <memory>

namespace tpm {

class GraphBase {
  protected:
    OpVec ops;
    TensorVec tensors;
    TensorVec inputs;
    TensorVec outputs;

  public:
    GraphBase() {}
    GraphBase(const GraphBase &) = delete;
    virtual ~GraphBase(); // owns its operators and tensors

    Tensor *tensor(const Dim &dims, Tensor::DataType dtype = Tensor::Float32);
    Tensor *tensor(const Dim &dims, const std::string &dtype);
    void addTensor(Tensor *t) { tensors.push_back(t); }
    TensorVec &getTensors() { return tensors; }
    OpVec &getOperators() { return ops; }
    const OpVec &getOperators() const { return ops; }
    TensorVec &getInputs() { return inputs; }
    const TensorVec &getInputs() const { return inputs; }
    TensorVec &getOutputs() { return outputs; }
    const TensorVec &getOutputs() const { return outputs; }

    // Fills inputOf / outputOf, predecessors / successors and the graph's
    // input and output lists from the operators' tensor lists.
    void updateConnection();
    void removeOps(OpVec &removed);
    // Operators in a topological order (Kahn, ties in insertion order).
    bool topoOrder(OpVec &order) const;
    // The reference reads and writes model files through its embedded Python plug-in
    // (src/Graph/graph.cc:1172-1187). Both are native here, on the protobuf wire format
    // directly: src/onnx_import.cc (one Graph builder call per node; the object must be a
    // Graph) and src/onnx_export.cc (one or a few nodes per operator, weights written with
    // their data). Each returns false with a message on stderr for what it cannot take.
    bool exportOnnx(const char *path);
    bool importOnnx(const char *net);
};

class Graph : public GraphBase {
  public:
    Graph() {}

    Operator *conv(Tensor *input, Tensor *weight, Tensor *output, int ph, int pw, int sh = 1,
                   int sw = 1, int dh = 1, int dw = 1, Tensor *bias = nullptr);
    Operator *conv(Tensor *input, Tensor *weight, int ph, int pw, int sh = 1, int sw = 1,
                   int dh = 1, int dw = 1, Tensor *bias = nullptr);
    Operator *conv(Tensor *input, Tensor *weight, Tensor *output, ConvOp::PaddingMode pm,
                   int sh = 1, int sw = 1, int dh = 1, int dw = 1, Tensor *bias = nullptr);
    Operator *conv(Tensor *input, Tensor *weight, ConvOp::PaddingMode pm, int sh = 1, int sw = 1,
                   int dh = 1, int dw = 1, Tensor *bias = nullptr);
    // Transposed convolution on NCHW input / [f, c, r, s] weight / NCHW output: the layout
    // transposes around the NHWC operator are part of what is built (include/graph.h:55-74).
    Tensor *setConvTransInput(Tensor *input);
    Tensor *setConvTransWeight(Tensor *weight);
    Tensor *setConvTransOutput(Tensor *outputTrans, Tensor *output = nullptr);
    Operator *convTrans(Tensor *input, Tensor *weight, Tensor *output, int ph, int pw, int sh = 1,
                        int sw = 1, int dh = 1, int dw = 1, int oph = 0, int opw = 0,
                        Tensor *bias = nullptr);
    Operator *convTrans(Tensor *input, Tensor *weight, Tensor *output,
                        ConvTransOp::PaddingMode pm, int sh = 1, int sw = 1, int dh = 1,
                        int dw = 1, int oph = 0, int opw = 0, Tensor *bias = nullptr);
    Operator *g2bmm(Tensor *A, Tensor *B, Tensor *C, int width, int dilation,
                    Tensor *bias = nullptr);
    Operator *g2bmm(Tensor *A, Tensor *B, int width, int dilation, Tensor *bias = nullptr);
    Operator *gbmml(Tensor *A, Tensor *B, Tensor *C, int dilation, Tensor *bias = nullptr);
    Operator *gbmml(Tensor *A, Tensor *B, int dilation, Tensor *bias = nullptr);
    Operator *conv3d(Tensor *input, Tensor *weight, Tensor *output, const Dim &pad,
                     const Dim &stride, const Dim &dilation, Tensor *bias = nullptr);
    Operator *matmul(Tensor *A, Tensor *B, Tensor *C, bool transA = false, bool transB = false,
                     Tensor *bias = nullptr);
    Operator *matmul(Tensor *A, Tensor *B, bool transA = false, bool transB = false,
                     Tensor *bias = nullptr);
    Operator *pad(Tensor *input, Tensor *output, const Dim &begin, const Dim &end);
    Operator *pad(Tensor *input, const Dim &begin, const Dim &end);
    Operator *slice(Tensor *input, Tensor *output, const Dim &begin, const Dim &end);
    Operator *slice(Tensor *input, const Dim &begin, const Dim &end);
    Operator *concat(const TensorVec &inputs, Tensor *output, int dim);
    Operator *concat(const TensorVec &inputs, int dim);
    Operator *split(Tensor *input, const TensorVec &outputs, int dim, int num);
    Operator *split(Tensor *input, int dim, int num);
    Operator *split(Tensor *input, const TensorVec &outputs, int dim, std::vector<int> sizes);
    Operator *split(Tensor *input, int dim, std::vector<int> sizes);
    Operator *transpose(Tensor *input, Tensor *output, int split, const Perm &after,
                        int factor = 2);
    Operator *transpose(Tensor *input, int split, const Perm &after, int factor = 2);
    Operator *flatten(Tensor *input, Tensor *output, int axis);
    Operator *extend(Tensor *input, Tensor *output, int dim, int num);
    Operator *extend(Tensor *input, int dim, int num);
    Operator *maxpool(Tensor *input, Tensor *output, int kh, int kw, int dh, int dw, int ph,
                      int pw, int sh, int sw);
    Operator *avgpool(Tensor *input, Tensor *output, int kh, int kw, int ph, int pw, int sh,
                      int sw);
    Operator *avgpool(Tensor *input, Tensor *output); // global
    Operator *add(const TensorVec &inputs, Tensor *output);
    Operator *add(const TensorVec &inputs);
    Operator *sub(Tensor *a, Tensor *b, Tensor *output);
    Operator *mul(const TensorVec &inputs, Tensor *output);
    Operator *mul(const TensorVec &inputs);
    Operator *div(Tensor *input0, Tensor *input1, Tensor *output);
    Operator *div(Tensor *input0, Tensor *input1);
    Operator *pow(Tensor *input, Tensor *output, int pow);
    Operator *pow(Tensor *input, int pow);
    Operator *gather(Tensor *data, Tensor *indices, Tensor *output, int axis);
    Operator *gather(Tensor *data, Tensor *indices, int axis);
    Operator *reduceMean(Tensor *input, Tensor *output, int axis);
    Operator *reduceMean(Tensor *input, int axis);
    Operator *batchnorm(Tensor *input, Tensor *scale, Tensor *bias, Tensor *mean, Tensor *var,
                        Tensor *output, float epsilon = 1e-05, float momentum = 0.9);
    Operator *batchnorm(Tensor *input, Tensor *scale, Tensor *bias, Tensor *mean, Tensor *var,
                        float epsilon = 1e-05, float momentum = 0.9);
    Operator *reshape(Tensor *input, Tensor *output);
    Operator *identity(Tensor *input, Tensor *output);
    Operator *relu(Tensor *input, Tensor *output);
    Operator *relu(Tensor *input);
    Operator *sigmoid(Tensor *input, Tensor *output);
    Operator *tanh(Tensor *input, Tensor *output);
    Operator *gelu(Tensor *input, Tensor *output);
    Operator *softmax(Tensor *input, Tensor *output, int axis);
    Operator *layernorm(Tensor *input, Tensor *output, Tensor *gamma, Tensor *beta,
                        float eps = 1e-5f);

    void setInputs(TensorVec v) { inputs = std::move(v); }
    void setOutputs(TensorVec v) { outputs = std::move(v); }
#ifdef PET_HAVE_NNET
    // A memory-bound operator given by an expression of the reference's nnet tree
    // (include/graph.h:176-180, src/Graph/graph.cc:603-613); only where that tree's
    // headers are on the include path.
    Operator *membound(const TensorVec &inputs, const TensorVec &outputs,
                       const std::vector<nnet::Tensor> &nnetInputs, nnet::Expr expr,
                       double exec_time, std::string hint = {}) {
        // 0.001 ms for the launch, as upstream
        double t = exec_time == 0 ? 0 : std::max(exec_time, 0.001);
        // the outputs are the caller's tensors (often another graph's): not adopted
        ops.push_back(new MemBoundOp(inputs, outputs, nnetInputs, expr, t, hint));
        return ops.back();
    }
#endif

    // Takes ownership of an operator built elsewhere (and of the outputs it created).
    Operator *own(Operator *op);
};

class SubGraph : public GraphBase {
    uint64_t hash = 2147483647;

  public:
    SubGraph() {}
    // Clones the operators and their tensors (tensors are matched by hash).
    explicit SubGraph(OpVec oplist);
    SubGraph(const SubGraph &rhs) : SubGraph(rhs.ops) {}

    // Runs every operator on the device in topological order.
    bool compute();
    // One output value; computes on the device whatever part of the graph has
    // not been computed yet. const like the reference's (the tensors it
    // updates are reached through pointers).
    const std::pair<bool, VType> compute(const Dim &point, size_t outputId = 0,
                                         bool getAllPos = false) const;
    // Re-wires the graph around a borrowed operator list whose tensors are the
    // first `ntensor` (0: all) of this graph's tensors; false when an operator
    // touches a tensor outside the graph (reference src/Graph/graph.cc:736-778).
    // This is how the mutation generator reuses one scratch graph for every
    // candidate it tries.
    bool resetOps(OpVec oplist, size_t ntensor = 0);
    void cleanConnection();
    int findTensor(Tensor *tensor, int ntensor = 0);
    // Seeds both graphs' inputs with the same data, runs both on the device
    // and compares every output element for equality.
    bool verification(SubGraph *mutant_graph, bool isFullComputing = true);
    // Sum of op->perf() over the operators, in ms.
    double perf(PerfEngine *pe, bool withPenalty = true);
    uint64_t getHash();
    // Key of the search engine's mutation archive: operator types, at level 1 also the
    // extents of their inputs (src/Graph/graph.cc:901-924).
    uint64_t getCacheIdx(int level);
    int print();
    int printBrief();
    int getComputeOps(OpVec &out);
    void resetComputed();
    // Gives the graph's inputs and outputs the identity (hash) of the given tensors, so
    // that a mutant can take the place of the subgraph it was derived from.
    int reset(std::vector<Tensor *> &input, std::vector<Tensor *> &output);
    // The operators of `ops` as `slave`, all others as `master` (both cloned).
    int split(std::shared_ptr<SubGraph> &master, std::shared_ptr<SubGraph> &slave,
              std::vector<Operator *> &ops);
    // This graph's operators plus the slave's, the slave's tensors replaced by this
    // graph's where their hashes agree.
    int merge(std::shared_ptr<SubGraph> &master, std::shared_ptr<SubGraph> &slave);
};

} // namespace tpm

