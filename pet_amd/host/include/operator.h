// Operators of the PET graph on the MI355X backend (role of the reference's
// include/operator.h). Same class names, constructor arguments and virtual
// interface for the operators on the contraction / layout path, so the
// mutators and the search engine can drive them unchanged; every compute()
// and perf() runs HIP kernels through the C ABI (pet_hip.h), never the host.
#pragma once
#include "common.h"
#include "perf.h"
#include "tensor.h"
#include "transpose.h"
#include <sstream>
// MemBoundOp is defined over the expression tree of the reference's search side
// (include/nnet/expr.h). That tree is not part of this backend: where its headers are on
// the include path (builds of the reference's mutators and search engine against this
// directory) the class exists, elsewhere nothing here depends on it.
#if __has_include("nnet/expr.h")
#define PET_HAVE_NNET 1
#include "nnet/expr.h"
#endif

namespace tpm {

class PerfEngine;

// While one of these lives (on this thread), an operator constructor that finds its operands
// invalid throws std::invalid_argument instead of asserting.
struct InvalidOperandsThrow {
    InvalidOperandsThrow();
    ~InvalidOperandsThrow();
    InvalidOperandsThrow(const InvalidOperandsThrow &) = delete;
};

class Operator {
  public:
    // Numbering as in the reference (include/operator.h:19-51); the ops this
    // backend does not execute are kept so type codes stay comparable.
    enum OpType {
        Unknown = 0,
        Conv = 100,
        Matmul,
        ConvTrans,
        G2BMM,
        GBMML,
        Pad,
        Slice,
        Concat,
        Split,
        Transpose,
        Extend,
        MaxPool,
        AvgPool,
        Add,
        Sub,
        Mul,
        Div,
        Pow,
        Gather,
        ReduceMean,
        Reshape,
        Identity,
        BatchNorm = 200,
        Softmax,
        Activation,
        Resize,
        MemBound = 300,
        Conv3d = 400, // not in the reference: ConvOp with a depth axis
        LayerNorm,    // not in the reference
    };
    static std::string getOpName(OpType t);

    enum ActType { None, Relu, Sigmoid, Tanh, Gelu /* Gelu is not in the reference */ };

    Operator() : guid(generateGuid()), hash(generateHash()), type(Unknown) {}
    explicit Operator(OpType type) : guid(generateGuid()), hash(generateHash()), type(type) {}
    Operator(OpType type, TensorVec inputs, TensorVec outputs = {})
        : guid(generateGuid()), hash(generateHash()), type(type), inputs(std::move(inputs)),
          outputs(std::move(outputs)) {}
    Operator(const Operator &rhs) : guid(generateGuid()), hash(rhs.hash), type(rhs.type) {}
    virtual ~Operator() {}

    bool isLinearOp() const { return type >= 100 && type < 200; }
    bool isElementWiseOp() const { return type >= 200 && type < 300; }
    bool isSplitOp() const { return type == Split; }
    bool isConcatOp() const { return type == Concat; }
    bool isComputeOp() const { return type == Conv || type == Matmul || type == Conv3d; }
    bool isTransposeOp() const { return type == Transpose; }
    bool isReshapeOp() const { return type == Reshape; }
    bool isMemBoundOp() const { return type == MemBound || type == Activation || type == Transpose; }

    bool isClear() const {
        return inputs.empty() && outputs.empty() && successors.empty() && predecessors.empty();
    }
    void clear() {
        inputs.clear();
        outputs.clear();
        successors.clear();
        predecessors.clear();
    }

    void setSuccessors(OpVec v) { successors = std::move(v); }
    void setPredecessors(OpVec v) { predecessors = std::move(v); }
    void addSuccessors(Operator *op) { successors.push_back(op); }
    void addPredecessors(Operator *op) { predecessors.push_back(op); }
    OpVec &getSuccessors() { return successors; }
    const OpVec &getSuccessors() const { return successors; }
    OpVec &getPredecessors() { return predecessors; }
    const OpVec &getPredecessors() const { return predecessors; }
    Operator *getPredecessor() { return predecessors.size() == 1 ? predecessors[0] : nullptr; }

    TensorVec &getInputs() { return inputs; }
    const TensorVec &getInputs() const { return inputs; }
    TensorVec &getOutputs() { return outputs; }
    const TensorVec &getOutputs() const { return outputs; }
    void setInputs(const TensorVec &v) { inputs = v; }
    void setOutputs(const TensorVec &v) { outputs = v; }
    Tensor *getInputs(size_t i) { return i < inputs.size() ? inputs[i] : nullptr; }
    Tensor *getOutput() const { return isSplitOp() || outputs.empty() ? nullptr : outputs[0]; }
    void addInput(Tensor *t) { inputs.push_back(t); }
    void addOutput(Tensor *t) { outputs.push_back(t); }

    // Time of one launch in ms on this GPU, hipEvent-timed on the backend
    // stream and memoised in the PerfEngine; INFINITY if the backend rejects
    // the shape.
    virtual double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) = 0;
    virtual Operator *clone() = 0;

    // Computes the outputs on the device. nullptr when the operator rejects
    // its shapes (same cases as the reference).
    virtual Tensor *compute();
    // Destination points -> (input ranges, closure that performs the
    // computation). The closure always runs the whole operator on the device:
    // there is no host arithmetic in this layer.
    virtual std::pair<std::vector<DimRange>, std::function<bool()>> compute(DimRange dr);
    virtual bool compute(const TensorVec &ins, const TensorVec &outs) {
        return computeShape(ins, outs) && compute() != nullptr;
    }

    virtual Dim computeShape() = 0;
    virtual bool computeShape(const TensorVec &ins, const TensorVec &outs);

    // Contractions only (Conv, Conv3d, Matmul): one launch of
    // out = finalAct(op(inputs) + bias + residual), residual and out laid out like
    // the operator's output. The graph runtime uses it to run "contraction, Add,
    // activation" as one operator. PET_HIP_ERR_UNSUPPORTED elsewhere.
    // flags: pet_hip_call_flags, what the graph runtime fuses across launches.
    virtual int launchFused(pet_hip_stream_t stream, const float *residual, ActType finalAct,
                            float *out, unsigned flags = 0);
    virtual bool canTakeResidual() const { return false; }
    // Contractions only: whether a launch adds partial sums into the output with
    // atomics, i.e. starts by writing the bias into all of it.
    virtual bool accumulates() const { return false; }

    virtual int numInputs() = 0;
    virtual int numOutputs() = 0;
    void print() const { std::cout << toString() << std::endl; }
    virtual std::string toString() const = 0;
    virtual std::string getName() const { return getOpName(type); }

    size_t getGuid() const { return guid; }
    uint64_t getHash() const { return hash; }
    OpType getType() const { return type; }

    virtual void inferSplittingPoints();
    virtual void getOptypeAttr(std::string &optype, std::map<std::string, std::string> &attr,
                               std::map<std::string, std::vector<int>> &extra) const;

    // Issues the operator's kernels on `stream` with the tensors' device
    // buffers (used by compute(), by perf() and by the graph runtime).
    // Returns a pet_hip_status.
    virtual int launch(pet_hip_stream_t stream) = 0;
    // For operators the emitter has no case of its own for: the C-ABI call that launches
    // the operator on stream `s` in an emitted program, `name` giving a tensor's variable
    // and `setup` taking lines that must precede the captured region. Empty: cannot be
    // emitted.
    virtual std::string emitLaunch(const std::function<std::string(const Tensor *)> &name,
                                   std::vector<std::string> &setup) const {
        (void)name;
        (void)setup;
        return "";
    }

  protected:
    virtual bool checkValid(const TensorVec &inputs) = 0;
    virtual void initHash() = 0;
    bool allocOutputs();
    // hipEvent timing of `launch` on the backend stream.
    double timeLaunches(int rounds, int warmupRounds);

    const size_t guid;
    uint64_t hash;
    OpType type;
    TensorVec inputs;
    TensorVec outputs;
    OpVec predecessors;
    OpVec successors;
};

// ---- Conv ---------------------------------------------------------------------
class ConvOp : public Operator {
  public:
    enum PaddingMode { Other, Same, Valid };

    ConvOp(Tensor *input, Tensor *weight, Tensor *output, int ph, int pw, int sh = 1, int sw = 1,
           int dh = 1, int dw = 1, Tensor *bias = nullptr, ActType act = None);
    ConvOp(Tensor *input, Tensor *weight, int ph, int pw, int sh = 1, int sw = 1, int dh = 1,
           int dw = 1, Tensor *bias = nullptr, ActType act = None);
    ConvOp(int ph, int pw, int sh = 1, int sw = 1, int dh = 1, int dw = 1, Tensor *bias = nullptr,
           ActType act = None);
    ConvOp(Tensor *input, Tensor *weight, Tensor *output, PaddingMode pm = Same, int sh = 1,
           int sw = 1, int dh = 1, int dw = 1, Tensor *bias = nullptr, ActType act = None);
    ConvOp(Tensor *input, Tensor *weight, PaddingMode pm = Same, int sh = 1, int sw = 1,
           int dh = 1, int dw = 1, Tensor *bias = nullptr, ActType act = None);
    ConvOp(PaddingMode pm = Same, int sh = 1, int sw = 1, int dh = 1, int dw = 1,
           Tensor *bias = nullptr, ActType act = None);
    ConvOp(const ConvOp &rhs);
    ConvOp *clone() override { return new ConvOp(*this); }

    Dim computeShape() override;
    Dim computeOutputPenalty(const Dim &p);
    double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) override;
    int launch(pet_hip_stream_t stream) override;
    int launchFused(pet_hip_stream_t stream, const float *residual, ActType finalAct,
                    float *out, unsigned flags = 0) override;
    // The same convolution with x read and / or y written through strides (NULL: the usual
    // layout): a row of Transposes next to it folded into its addressing by the graph runtime.
    int launchView(pet_hip_stream_t stream, const float *x, const pet_hip_conv_view *xView,
                   float *y, const pet_hip_conv_view *yView, unsigned flags);
    bool accumulates() const override;
    bool canTakeResidual() const override { return act == None; }
    std::string toString() const override;
    int numInputs() override { return 2; }
    int numOutputs() override { return 1; }

    Tensor *getBias() const { return bias; }
    void setAct(ActType a) { act = a; }
    ActType getAct() const { return act; }
    // Which of the backend's PET_HIP_CONV_ALGO_COUNT ways of sharing out the K loop the
    // launches use; perf() leaves the fastest one here (0: the library's cost model),
    // CodeEngine takes it from an imported PerfEngine (the role of ConvResult::algo and
    // PerfEngine::getConvAlgo in the reference, src/Graph/code_engine.cc:874-878).
    void setAlgo(int a) { algo = a; }
    int getAlgo() const { return algo; }
    bool same(const ConvOp &rhs);
    PaddingMode getPaddingMode() { return padding; }
    int getDh() const { return dh; }
    int getDw() const { return dw; }
    int getPh() const { return ph; }
    int getPw() const { return pw; }
    int getSh() const { return sh; }
    int getSw() const { return sw; }
    ConvArgs getArgs(int withPenalty) const;

  private:
    bool checkValid(const TensorVec &inputs) override;
    void initHash() override;
    void setPaddingMode();
    // output extents for the current padding mode; updates ph / pw in the
    // Same / Valid modes
    void outputExtent(int h, int w, int r, int s, int &oh, int &ow);

    int ph = 0, pw = 0, sh, sw, dh, dw;
    Tensor *bias; // side pointer, not a graph edge
    ActType act;
    PaddingMode padding;
    int algo = 0;
};

// ---- Conv3d (extension: the reference has no 3-D convolution) -----------------
class Conv3dOp : public Operator {
  public:
    Conv3dOp(Tensor *input, Tensor *weight, Tensor *output, const Dim &pad, const Dim &stride,
             const Dim &dilation, Tensor *bias = nullptr, ActType act = None);
    Conv3dOp(const Conv3dOp &rhs);
    ~Conv3dOp() override;
    Conv3dOp *clone() override { return new Conv3dOp(*this); }
    // Weight preprocessing, run once by whoever treats the filters as constants
    // (CodeEngine before it captures a graph): keeps a kt-major copy of the
    // filters that launch() then reads through pet_hip_conv3d_packed_f32 for as
    // long as the weight tensor is not written again. False (and no copy) when
    // the backend has no such form for this shape.
    bool prepackFilters(pet_hip_stream_t stream);
    bool usesPackedFilters() const;
    Dim computeShape() override;
    double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) override;
    int launch(pet_hip_stream_t stream) override;
    int launchFused(pet_hip_stream_t stream, const float *residual, ActType finalAct,
                    float *out, unsigned flags = 0) override;
    bool accumulates() const override;
    bool canTakeResidual() const override { return act == None; }
    std::string toString() const override;
    int numInputs() override { return 2; }
    int numOutputs() override { return 1; }
    void setAct(ActType a) { act = a; }
    ActType getAct() const { return act; }
    // as ConvOp::setAlgo; perf() leaves the fastest of the backend's algorithms here
    void setAlgo(int a) { algo = a; }
    int getAlgo() const { return algo; }
    Tensor *getBias() const { return bias; }
    const Dim &getPad() const { return pad; }
    const Dim &getStride() const { return stride; }
    const Dim &getDilation() const { return dilation; }

  private:
    bool checkValid(const TensorVec &inputs) override;
    void initHash() override;
    Dim pad, stride, dilation; // (t, h, w)
    Tensor *bias;
    ActType act;
    float *packed = nullptr;     // kt-major filters, owned
    size_t packedElems = 0;
    uint64_t packedVersion = 0;  // weight tensor's dataVersion() the copy was made from
    int algo = 0;
};

// ---- Matmul -------------------------------------------------------------------
class MatmulOp : public Operator {
  public:
    MatmulOp(Tensor *A, Tensor *B, Tensor *C, bool transA = false, bool transB = false,
             Tensor *bias = nullptr, ActType act = None);
    MatmulOp(Tensor *A, Tensor *B, bool transA = false, bool transB = false,
             Tensor *bias = nullptr, ActType act = None);
    MatmulOp(bool transA = false, bool transB = false, Tensor *bias = nullptr, ActType act = None);
    MatmulOp(const MatmulOp &rhs)
        : Operator(rhs), transA(rhs.transA), transB(rhs.transB), bias(rhs.bias), act(rhs.act),
          algo(rhs.algo) {}
    // as ConvOp::setAlgo (MatmulResult::algo, PerfEngine::getMatmulAlgo)
    void setAlgo(int a) { algo = a; }
    int getAlgo() const { return algo; }
    MatmulOp *clone() override { return new MatmulOp(*this); }
    // One output point -> the input points it depends on; the closure runs the
    // whole operator on the device.
    std::pair<std::vector<DimRange>, std::function<bool()>> compute(DimRange dr) override;
    using Operator::compute;

    Dim computeShape() override;
    double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) override;
    int launch(pet_hip_stream_t stream) override;
    int launchFused(pet_hip_stream_t stream, const float *residual, ActType finalAct,
                    float *out, unsigned flags = 0) override;
    bool accumulates() const override;
    bool canTakeResidual() const override { return act == None; }
    std::string toString() const override;
    int numInputs() override { return 2; }
    int numOutputs() override { return 1; }
    Tensor *getBias() const { return bias; }
    // Set by the graph runtime when the lhs is `count` copies of one [1, m, k] tensor stacked
    // on dim 0 (an Extend, or a Concat of the same tensor: the batch-matmul merge of
    // src/Mutant/generator.cc:1495-1552 applied to projections of one input): the launch then
    // reads that tensor for every batch entry and the stacked copy is never made.
    void setSharedLhs(Tensor *src) { sharedLhs = src; }
    Tensor *getSharedLhs() const { return sharedLhs; }
    // A bias of b * n values is one row per batch entry (the merged projections' biases).
    bool biasPerBatch() const;
    unsigned operandFlags() const;
    void setAct(ActType a) { act = a; }
    ActType getAct() const { return act; }
    bool getTransA() const { return transA; }
    bool getTransB() const { return transB; }
    MatmulArgs getArgs() const;
    void dimExtend(Tensor *t); // 2-D tensors get a leading 1

  private:
    bool checkValid(const TensorVec &inputs) override;
    void initHash() override;
    void markWeight(Tensor *A, Tensor *B);
    bool transA, transB;
    Tensor *bias;
    ActType act;
    int algo = 0;
    Tensor *sharedLhs = nullptr;
};

// ---- ConvTrans -----------------------------------------------------------------------
// Transposed convolution in the reference's operator-level layout: input NHWF [n,h,w,f],
// weight RSFC [r,s,f,c], output NHWC [n,oh,ow,c] (include/operator.h:466-612,
// src/Graph/operator.cc:866-1100). Graph::convTrans takes NCHW tensors and puts the
// layout transposes around it, as the reference's builder does.
class ConvTransOp : public Operator {
  public:
    enum PaddingMode { Other, Same, Valid };

    ConvTransOp(Tensor *input, Tensor *weight, Tensor *output, int ph, int pw, int sh = 1,
                int sw = 1, int dh = 1, int dw = 1, int oph = 1, int opw = 1,
                Tensor *bias = nullptr, ActType act = None);
    ConvTransOp(Tensor *input, Tensor *weight, int ph, int pw, int sh = 1, int sw = 1, int dh = 1,
                int dw = 1, int oph = 0, int opw = 0, Tensor *bias = nullptr, ActType act = None);
    ConvTransOp(int ph, int pw, int sh = 1, int sw = 1, int dh = 1, int dw = 1, int oph = 0,
                int opw = 0, Tensor *bias = nullptr, ActType act = None);
    ConvTransOp(Tensor *input, Tensor *weight, Tensor *output, PaddingMode pm = Same, int sh = 1,
                int sw = 1, int dh = 1, int dw = 1, int oph = 0, int opw = 0,
                Tensor *bias = nullptr, ActType act = None);
    ConvTransOp(Tensor *input, Tensor *weight, PaddingMode pm = Same, int sh = 1, int sw = 1,
                int dh = 1, int dw = 1, int oph = 1, int opw = 1, Tensor *bias = nullptr,
                ActType act = None);
    ConvTransOp(PaddingMode pm = Same, int sh = 1, int sw = 1, int dh = 1, int dw = 1,
                int oph = 0, int opw = 0, Tensor *bias = nullptr, ActType act = None);
    ConvTransOp(const ConvTransOp &rhs);
    ConvTransOp *clone() override { return new ConvTransOp(*this); }

    Dim computeShape() override;
    double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) override;
    int launch(pet_hip_stream_t stream) override;
    std::string toString() const override;
    int numInputs() override { return 2; }
    int numOutputs() override { return 1; }
    Tensor *getBias() const { return bias; }
    void setAct(ActType a) { act = a; }
    ActType getAct() const { return act; }
    bool same(const ConvTransOp &rhs);
    PaddingMode getPaddingMode() { return padding; }
    int getDh() const { return dh; }
    int getDw() const { return dw; }
    int getPh() const { return ph; }
    int getPw() const { return pw; }
    int getSh() const { return sh; }
    int getSw() const { return sw; }
    int getOph() const { return oph; }
    int getOpw() const { return opw; }
    // n, c, h, w, f, r, s, ph, pw, sh, sw, dh, dw, g, bias, act with c the output
    // channels and f the input features (include/operator.h:584-599)
    ConvArgs getArgs(int withPenalty) const;

  private:
    bool checkValid(const TensorVec &inputs) override;
    void initHash() override;
    void setPaddingMode();
    int ph = 0, pw = 0, sh, sw, dh, dw, oph, opw;
    Tensor *bias; // not part of the graph connections
    ActType act;
    PaddingMode padding;
};

// ---- band matrix products ---------------------------------------------------------------
// G2BMM (general x general -> band) and GBMML (band x general -> general) are the
// sliding-window attention products. The reference has no host evaluation for them
// (src/Graph/operator.cc:1355-1391, 1498-1527) and runs two generated kernels fixed to
// one shape (include/custom_ops.cuh:3538-3559); here they run on the device for any
// shape, by the definitions of src/nnet/iterator_table.cc:596-630.
typedef std::tuple<int, int, int, int, int> G2BMMGBMMLArgs; // b, m, k, width, dilation

class G2BMMOp : public Operator {
  public:
    G2BMMOp(Tensor *A, Tensor *B, Tensor *C, int width, int dilation, Tensor *bias = nullptr,
            ActType act = None);
    G2BMMOp(Tensor *A, Tensor *B, int width, int dilation, Tensor *bias = nullptr,
            ActType act = None);
    G2BMMOp(int width, int dilation, Tensor *bias = nullptr, ActType act = None);
    G2BMMOp(const G2BMMOp &rhs)
        : Operator(rhs), width(rhs.width), dilation(rhs.dilation), bias(rhs.bias), act(rhs.act) {}
    G2BMMOp *clone() override { return new G2BMMOp(*this); }
    Dim computeShape() override; // [b, m, 2 * width + 1]
    double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) override;
    int launch(pet_hip_stream_t stream) override;
    std::string toString() const override;
    int numInputs() override { return 2; }
    int numOutputs() override { return 1; }
    int getWidth() const { return width; }
    int getDilation() const { return dilation; }
    Tensor *getBias() const { return bias; }
    void setAct(ActType a) { act = a; }
    ActType getAct() const { return act; }
    G2BMMGBMMLArgs getArgs() const;

  private:
    bool checkValid(const TensorVec &inputs) override;
    void initHash() override;
    int width, dilation;
    Tensor *bias; // not part of the graph connections
    ActType act;
};

class GBMMLOp : public Operator {
  public:
    GBMMLOp(Tensor *A, Tensor *B, Tensor *C, int dilation, Tensor *bias = nullptr,
            ActType act = None);
    GBMMLOp(Tensor *A, Tensor *B, int dilation, Tensor *bias = nullptr, ActType act = None);
    GBMMLOp(int dilation, Tensor *bias = nullptr, ActType act = None);
    GBMMLOp(const GBMMLOp &rhs)
        : Operator(rhs), dilation(rhs.dilation), bias(rhs.bias), act(rhs.act) {}
    GBMMLOp *clone() override { return new GBMMLOp(*this); }
    Dim computeShape() override; // [b, m, k] from A[b, m, 2w+1], B[b, m, k]
    double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) override;
    int launch(pet_hip_stream_t stream) override;
    std::string toString() const override;
    int numInputs() override { return 2; }
    int numOutputs() override { return 1; }
    int getDilation() const { return dilation; }
    Tensor *getBias() const { return bias; }
    void setAct(ActType a) { act = a; }
    ActType getAct() const { return act; }
    G2BMMGBMMLArgs getArgs() const;

  private:
    bool checkValid(const TensorVec &inputs) override;
    void initHash() override;
    int dilation;
    Tensor *bias;
    ActType act;
};

// ---- Pad / Slice --------------------------------------------------------------
class PadOp : public Operator {
  public:
    PadOp(Tensor *input, Tensor *output, const Dim &begin, const Dim &end);
    PadOp(Tensor *input, const Dim &begin, const Dim &end);
    PadOp(const Dim &begin, const Dim &end);
    PadOp(const PadOp &rhs) : Operator(rhs), begin(rhs.begin), end(rhs.end) {}
    PadOp *clone() override { return new PadOp(*this); }
    Dim computeShape() override;
    double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) override;
    int launch(pet_hip_stream_t stream) override;
    std::string toString() const override;
    int numInputs() override { return 1; }
    int numOutputs() override { return 1; }
    const Dim &getBegin() const { return begin; }
    const Dim &getEnd() const { return end; }

  private:
    bool checkValid(const TensorVec &inputs) override;
    void initHash() override;
    Dim begin, end;
};

class SliceOp : public Operator {
  public:
    SliceOp(Tensor *input, Tensor *output, const Dim &begin, const Dim &end);
    SliceOp(Tensor *input, const Dim &begin, const Dim &end);
    SliceOp(const Dim &begin, const Dim &end);
    SliceOp(const SliceOp &rhs) : Operator(rhs), begin(rhs.begin), end(rhs.end) {}
    SliceOp *clone() override { return new SliceOp(*this); }
    Dim computeShape() override;
    double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) override;
    int launch(pet_hip_stream_t stream) override;
    std::string toString() const override;
    int numInputs() override { return 1; }
    int numOutputs() override { return 1; }
    const Dim &getBegin() const { return begin; }
    const Dim &getEnd() const { return end; }

  private:
    bool checkValid(const TensorVec &inputs) override;
    void initHash() override;
    Dim begin, end;
};

// ---- Concat / Split -------------------------------------------------------------
class ConcatOp : public Operator {
  public:
    ConcatOp(TensorVec inputs, int dim);
    ConcatOp(TensorVec inputs, Tensor *output, int dim);
    explicit ConcatOp(int dim);
    ConcatOp(const ConcatOp &rhs) : Operator(rhs), dim(rhs.dim) {}
    ConcatOp *clone() override { return new ConcatOp(*this); }
    // One output point -> the input points it depends on; the closure runs the
    // whole operator on the device.
    std::pair<std::vector<DimRange>, std::function<bool()>> compute(DimRange dr) override;
    using Operator::compute;
    Dim computeShape() override;
    double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) override;
    int launch(pet_hip_stream_t stream) override;
    std::string toString() const override;
    int numInputs() override { return (int)inputs.size(); }
    int numOutputs() override { return 1; }
    int getDim() const { return dim; }

  private:
    bool checkValid(const TensorVec &inputs) override;
    void initHash() override;
    int dim;
};

class SplitOp : public Operator {
  public:
    SplitOp(Tensor *input, int dim, int num);
    SplitOp(Tensor *input, int dim, const std::vector<int> &sizes);
    SplitOp(Tensor *input, const TensorVec &outputs, int dim, const std::vector<int> &sizes);
    SplitOp(int dim, int num);
    SplitOp(int dim, const std::vector<int> &sizes);
    SplitOp(const SplitOp &rhs) : Operator(rhs), dim(rhs.dim), num(rhs.num), sizes(rhs.sizes) {}
    SplitOp *clone() override { return new SplitOp(*this); }

    Tensor *compute() override; // returns outputs[0] (the reference asserts here)
    TensorVec computeV();
    using Operator::compute;
    // Point `dr` of output `idx` -> the input point it is copied from
    // (reference src/Graph/operator.cc:2027-2045). The closure splits the
    // whole tensor on the device.
    std::pair<std::vector<DimRange>, std::function<bool()>> compute(size_t idx, DimRange dr);
    Dim computeShape() override;            // dims of output 0
    std::vector<Dim> computeShapeV();       // ratio rule; empty when not divisible
    bool computeShape(const TensorVec &ins, const TensorVec &outs) override;
    double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) override;
    int launch(pet_hip_stream_t stream) override;
    std::string toString() const override;
    int numInputs() override { return 1; }
    int numOutputs() override { return (int)outputs.size(); }
    int getDim() const { return dim; }
    const std::vector<int> &getSizes() const { return sizes; }

  private:
    bool checkValid(const TensorVec &) override { return true; }
    void initHash() override;
    int dim, num;
    std::vector<int> sizes; // ratios of the split dim
};

// ---- Transpose ------------------------------------------------------------------
class PermItem {
    friend class Perm;
    std::vector<int> items;

  public:
    PermItem(int i) : items({i}) {}
    PermItem(std::initializer_list<int> lst) : items(lst) {}
    PermItem(const std::vector<int> &lst) : items(lst) {}
    bool isSingle() const { return items.size() == 1; }
    int getSingle() const { return items[0]; }
    std::vector<int> &getVec() { return items; }
    const std::vector<int> &getVec() const { return items; }
    std::string toString() const;
};

class Perm {
    std::vector<PermItem> perm;

  public:
    Perm(std::initializer_list<PermItem> perm) : perm(perm) {}
    Perm(const std::vector<PermItem> &perm) : perm(perm) {}
    std::vector<int> asVector() const;
    std::vector<PermItem> &getPerm() { return perm; }
    const std::vector<PermItem> &getPerm() const { return perm; }
    PermItem &operator[](size_t i) { return perm[i]; }
    const PermItem &operator[](size_t i) const { return perm[i]; }
    size_t size() const { return perm.size(); }
    std::string toString() const;
};

class TransposeOp : public Operator {
  public:
    enum TransType { NoneType, N2H, N2W, H2N, W2N, C2H, C2W, D2H, D2W };
    enum TransPos { NonePos, Pre, Post };

    TransposeOp(Tensor *input, Tensor *output, const Perm &before, const Perm &after,
                int factor = 2, TransType trans_type = NoneType);
    // In `after`, -1 names the dim the split introduces.
    TransposeOp(Tensor *input, Tensor *output, int split, const Perm &after, int factor = 2,
                TransType trans_type = NoneType);
    TransposeOp(Tensor *input, int split, const Perm &after, int factor = 2,
                TransType trans_type = NoneType);
    TransposeOp(int split, const Perm &after, int factor = 2, TransType trans_type = NoneType);
    TransposeOp(const TransposeOp &rhs);
    TransposeOp *clone() override { return new TransposeOp(*this); }
    // One output point -> the input points it depends on; the closure runs the
    // whole operator on the device.
    std::pair<std::vector<DimRange>, std::function<bool()>> compute(DimRange dr) override;
    using Operator::compute;

    Dim computeShape() override;
    double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) override;
    int launch(pet_hip_stream_t stream) override;
    std::string toString() const override;
    int numInputs() override { return 1; }
    int numOutputs() override { return 1; }

    // Micro-op lowering with the boundary-correction parameters: a Pre H2N/W2N
    // split carries `padding` halo rows (copys), the matching Post fuse drops
    // them (dels); a Pre N2H/N2W fuse inserts zero rows (pad), the Post split
    // skips them (extr).
    std::vector<std::shared_ptr<TransBasic>> getTTParam() const;

    void setPos(TransPos pos) { trans_pos = pos; }
    TransPos getPos() const { return trans_pos; }
    void setType(TransType t) { trans_type = t; }
    TransType getType() const { return trans_type; }
    std::pair<int, int> getPaddingSize() const { return {padding_h, padding_w}; }
    // With a non-zero padding size the operator runs its corrected form and
    // its output shape changes accordingly.
    void setPaddingSize(int h, int w) {
        padding_h = h;
        padding_w = w;
    }
    std::pair<Perm, Perm> getBeforeAndAfter() { return {before, after}; }
    int getSplit() const { return split; }
    int getFactor() const { return factor; }

  private:
    bool checkValid(const TensorVec &inputs) override;
    void initHash() override;
    void setParam(int dimSz);
    bool flatDims(Dim &flat) const; // false when the split does not divide
    bool corrected() const;

    Perm before, after;
    int split, factor;
    TransType trans_type;
    TransPos trans_pos = NonePos;
    int padding_h = 0, padding_w = 0;
};

// ---- Extend ---------------------------------------------------------------------
class ExtendOp : public Operator {
  public:
    ExtendOp(Tensor *input, Tensor *output, int dim, int num = 1);
    ExtendOp(Tensor *input, int dim, int num);
    ExtendOp(int dim, int num);
    ExtendOp(const ExtendOp &rhs) : Operator(rhs), dim(rhs.dim), num(rhs.num) {}
    ExtendOp *clone() override { return new ExtendOp(*this); }
    // One output point -> the input points it depends on; the closure runs the
    // whole operator on the device.
    std::pair<std::vector<DimRange>, std::function<bool()>> compute(DimRange dr) override;
    using Operator::compute;
    Dim computeShape() override;
    double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) override;
    int launch(pet_hip_stream_t stream) override;
    std::string toString() const override;
    int numInputs() override { return 1; }
    int numOutputs() override { return 1; }
    int getDim() const { return dim; }
    int getNum() const { return num; }

  private:
    bool checkValid(const TensorVec &) override { return true; }
    void initHash() override;
    int dim, num;
};

// ---- element-wise: Add / Sub / Mul / Div (flat-modulo broadcast) ------------------
class EltwiseOp : public Operator {
  public:
    EltwiseOp(OpType type, TensorVec inputs, Tensor *output);
    explicit EltwiseOp(OpType type) : Operator(type) { initHash(); }
    EltwiseOp(const EltwiseOp &rhs) : Operator(rhs) {}
    Dim computeShape() override;
    double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) override;
    int launch(pet_hip_stream_t stream) override;
    std::string toString() const override;
    int numInputs() override { return type == Sub || type == Div ? 2 : (int)inputs.size(); }
    int numOutputs() override { return 1; }
    // One output point -> the input points it depends on; the closure runs the
    // whole operator on the device.
    std::pair<std::vector<DimRange>, std::function<bool()>> compute(DimRange dr) override;
    using Operator::compute;
    bool computeShape(const TensorVec &ins, const TensorVec &outs) override;

  protected:
    bool checkValid(const TensorVec &inputs) override;
    void initHash() override;
};

class AddOp : public EltwiseOp {
  public:
    AddOp(TensorVec inputs, Tensor *output) : EltwiseOp(Add, std::move(inputs), output) {}
    explicit AddOp(TensorVec inputs) : EltwiseOp(Add, std::move(inputs), nullptr) {}
    AddOp() : EltwiseOp(Add) {}
    AddOp *clone() override { return new AddOp(*this); }
};

class SubOp : public EltwiseOp {
  public:
    SubOp(Tensor *a, Tensor *b, Tensor *output = nullptr) : EltwiseOp(Sub, {a, b}, output) {}
    SubOp() : EltwiseOp(Sub) {}
    SubOp *clone() override { return new SubOp(*this); }
};

class MulOp : public EltwiseOp {
  public:
    MulOp(TensorVec inputs, Tensor *output) : EltwiseOp(Mul, std::move(inputs), output) {}
    explicit MulOp(TensorVec inputs) : EltwiseOp(Mul, std::move(inputs), nullptr) {}
    MulOp() : EltwiseOp(Mul) {}
    MulOp *clone() override { return new MulOp(*this); }
};

// Division proper: the reference's CPU body subtracts (src/Graph/operator.cc:3259)
// and it has no GPU emitter for Div.
class DivOp : public EltwiseOp {
  public:
    DivOp(TensorVec inputs, Tensor *output) : EltwiseOp(Div, std::move(inputs), output) {}
    explicit DivOp(TensorVec inputs) : EltwiseOp(Div, std::move(inputs), nullptr) {}
    DivOp() : EltwiseOp(Div) {}
    DivOp *clone() override { return new DivOp(*this); }
};

// x multiplied up `pow` times from 1 (src/Graph/operator.cc:3315-3343).
class PowOp : public Operator {
  public:
    PowOp(Tensor *input, Tensor *output, int pow);
    PowOp(Tensor *input, int pow);
    explicit PowOp(int pow);
    PowOp(const PowOp &rhs) : Operator(rhs), pow(rhs.pow) {}
    PowOp *clone() override { return new PowOp(*this); }
    Dim computeShape() override;
    double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) override;
    int launch(pet_hip_stream_t stream) override;
    std::string toString() const override;
    int numInputs() override { return 1; }
    int numOutputs() override { return 1; }
    int getPow() const { return pow; }
    std::pair<std::vector<DimRange>, std::function<bool()>> compute(DimRange dr) override;
    using Operator::compute;

  private:
    bool checkValid(const TensorVec &ins) override { return ins.size() == 1 && ins[0]; }
    void initHash() override;
    int pow;
};

// Inference batch normalisation, channel = dim 1 (src/Graph/operator.cc:2660-2715).
// scale / bias / mean / var are side tensors of [channels], like a conv bias.
class BatchNormOp : public Operator {
  public:
    BatchNormOp(Tensor *input, Tensor *scale, Tensor *bias, Tensor *mean, Tensor *var,
                Tensor *output, float epsilon = 1e-05, float momentum = 0.9);
    BatchNormOp(Tensor *input, Tensor *scale, Tensor *bias, Tensor *mean, Tensor *var,
                float epsilon = 1e-05, float momentum = 0.9);
    BatchNormOp(Tensor *scale, Tensor *bias, Tensor *mean, Tensor *var, float epsilon = 1e-05,
                float momentum = 0.9);
    BatchNormOp(const BatchNormOp &rhs)
        : Operator(rhs), epsilon(rhs.epsilon), momentum(rhs.momentum), scale(rhs.scale),
          bias(rhs.bias), mean(rhs.mean), var(rhs.var) {}
    BatchNormOp *clone() override { return new BatchNormOp(*this); }
    Dim computeShape() override;
    double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) override;
    int launch(pet_hip_stream_t stream) override;
    std::string toString() const override;
    int numInputs() override { return 1; }
    int numOutputs() override { return 1; }
    Tensor *getScale() const { return scale; }
    Tensor *getBias() const { return bias; }
    Tensor *getMean() const { return mean; }
    Tensor *getVar() const { return var; }
    float getEpsilon() const { return epsilon; }
    std::pair<std::vector<DimRange>, std::function<bool()>> compute(DimRange dr) override;
    using Operator::compute;

  private:
    bool checkValid(const TensorVec &ins) override;
    void initHash() override;
    float epsilon, momentum;
    Tensor *scale, *bias, *mean, *var;
};

// out[j..., p..., q...] = data[p..., indices[j...], q...]: the index dims lead the
// output (src/Graph/operator.cc:3396-3428). Indices travel as fp32 values holding
// integers, like every tensor of this host layer.
class GatherOp : public Operator {
  public:
    GatherOp(Tensor *data, Tensor *indices, Tensor *output, int axis);
    GatherOp(Tensor *data, Tensor *indices, int axis);
    GatherOp() : Operator(Gather), axis(0) { initHash(); }
    GatherOp(const GatherOp &rhs) : Operator(rhs), axis(rhs.axis) {}
    GatherOp *clone() override { return new GatherOp(*this); }
    Dim computeShape() override;
    double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) override;
    int launch(pet_hip_stream_t stream) override;
    std::string toString() const override;
    int numInputs() override { return 2; }
    int numOutputs() override { return 1; }
    int getAxis() const { return axis; }

  private:
    bool checkValid(const TensorVec &ins) override;
    void initHash() override;
    int axis;
};

// Mean over one axis, which stays in the shape as 1 (src/Graph/operator.cc:3430-3458).
class ReduceMeanOp : public Operator {
  public:
    ReduceMeanOp(Tensor *input, Tensor *output, int axis);
    ReduceMeanOp(Tensor *input, int axis);
    ReduceMeanOp() : Operator(ReduceMean), axis(0) { initHash(); }
    ReduceMeanOp(const ReduceMeanOp &rhs) : Operator(rhs), axis(rhs.axis) {}
    ReduceMeanOp *clone() override { return new ReduceMeanOp(*this); }
    Dim computeShape() override;
    double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) override;
    int launch(pet_hip_stream_t stream) override;
    std::string toString() const override;
    int numInputs() override { return 1; }
    int numOutputs() override { return 1; }
    int getAxis() const { return axis; }

  private:
    bool checkValid(const TensorVec &ins) override;
    void initHash() override;
    int axis;
};

// ---- single-input ops without a reference CPU compute ----------------------------
class ActivationOp : public Operator {
  public:
    ActivationOp(Tensor *input, Tensor *output, ActType act);
    ActivationOp(Tensor *input, ActType act);
    explicit ActivationOp(ActType act);
    ActivationOp(const ActivationOp &rhs) : Operator(rhs), actType(rhs.actType) {}
    ActivationOp *clone() override { return new ActivationOp(*this); }
    Dim computeShape() override;
    double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) override;
    int launch(pet_hip_stream_t stream) override;
    std::string toString() const override;
    int numInputs() override { return 1; }
    int numOutputs() override { return 1; }
    ActType getActType() const { return actType; }

  private:
    bool checkValid(const TensorVec &) override { return true; }
    void initHash() override;
    ActType actType;
};

// Max / average pooling (one class, as the two differ in one flag).
class PoolOp : public Operator {
  public:
    PoolOp(OpType type, Tensor *input, Tensor *output, int kh, int kw, int dh, int dw, int ph,
           int pw, int sh, int sw);
    PoolOp(const PoolOp &rhs);
    PoolOp *clone() override { return new PoolOp(*this); }
    Dim computeShape() override;
    double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) override;
    int launch(pet_hip_stream_t stream) override;
    // flags: PET_HIP_CALL_X_RELU only (the producer's ReLU applied on the way in)
    int launchFused(pet_hip_stream_t stream, const float *residual, ActType finalAct, float *out,
                    unsigned flags) override;
    std::string toString() const override;
    int numInputs() override { return 1; }
    int numOutputs() override { return 1; }
    PoolArgs getArgs() const { return PoolArgs{kh, kw, ph, pw, sh, sw, dh, dw}; }

  private:
    bool checkValid(const TensorVec &inputs) override;
    void initHash() override;
    int kh, kw, dh, dw, ph, pw, sh, sw;
};

class MaxPoolOp : public PoolOp {
  public:
    MaxPoolOp(Tensor *input, Tensor *output, int kh, int kw, int dh, int dw, int ph, int pw,
              int sh, int sw)
        : PoolOp(MaxPool, input, output, kh, kw, dh, dw, ph, pw, sh, sw) {}
    // Output tensor made by the operator (reference include/operator.h:1332).
    MaxPoolOp(Tensor *input, int kh, int kw, int dh, int dw, int ph, int pw, int sh, int sw)
        : MaxPoolOp(input, new Tensor(), kh, kw, dh, dw, ph, pw, sh, sw) {}
};

class AvgPoolOp : public PoolOp {
  public:
    AvgPoolOp(Tensor *input, Tensor *output, int kh, int kw, int ph, int pw, int sh, int sw)
        : PoolOp(AvgPool, input, output, kh, kw, 1, 1, ph, pw, sh, sw) {}
    // Output tensor made by the operator (reference include/operator.h:1411).
    AvgPoolOp(Tensor *input, int kh, int kw, int ph, int pw, int sh, int sw)
        : AvgPoolOp(input, new Tensor(), kh, kw, ph, pw, sh, sw) {}
    // global average pool
    AvgPoolOp(Tensor *input, Tensor *output);
};

class SoftmaxOp : public Operator {
  public:
    SoftmaxOp(Tensor *input, Tensor *output, int axis);
    SoftmaxOp(const SoftmaxOp &rhs) : Operator(rhs), axis(rhs.axis) {}
    int getAxis() const { return axis; }
    SoftmaxOp *clone() override { return new SoftmaxOp(*this); }
    Dim computeShape() override;
    double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) override;
    int launch(pet_hip_stream_t stream) override;
    std::string toString() const override;
    int numInputs() override { return 1; }
    int numOutputs() override { return 1; }

  private:
    bool checkValid(const TensorVec &inputs) override;
    void initHash() override;
    int axis; // must be the last axis
};

class LayerNormOp : public Operator {
  public:
    LayerNormOp(Tensor *input, Tensor *output, Tensor *gamma, Tensor *beta, float eps = 1e-5f);
    LayerNormOp(const LayerNormOp &rhs)
        : Operator(rhs), gamma(rhs.gamma), beta(rhs.beta), eps(rhs.eps) {}
    LayerNormOp *clone() override { return new LayerNormOp(*this); }
    Dim computeShape() override;
    double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) override;
    int launch(pet_hip_stream_t stream) override;
    std::string toString() const override;
    int numInputs() override { return 1; }
    int numOutputs() override { return 1; }
    Tensor *getGamma() const { return gamma; }
    Tensor *getBeta() const { return beta; }
    float getEps() const { return eps; }

  private:
    bool checkValid(const TensorVec &) override { return true; }
    void initHash() override;
    Tensor *gamma, *beta; // side pointers like a conv bias
    float eps;
};

// Reshape / Identity: a copy with the output's dims (element count must match).
class ReshapeOp : public Operator {
  public:
    ReshapeOp(Tensor *input, Tensor *output);
    ReshapeOp(const ReshapeOp &rhs) : Operator(rhs) {}
    ReshapeOp *clone() override { return new ReshapeOp(*this); }
    Dim computeShape() override;
    double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) override;
    int launch(pet_hip_stream_t stream) override;
    std::string toString() const override;
    int numInputs() override { return 1; }
    int numOutputs() override { return 1; }

  protected:
    ReshapeOp(OpType type, Tensor *input, Tensor *output);
    bool checkValid(const TensorVec &inputs) override;
    void initHash() override;
};

class IdentityOp : public ReshapeOp {
  public:
    IdentityOp(Tensor *input, Tensor *output) : ReshapeOp(Identity, input, output) {}
    IdentityOp *clone() override { return new IdentityOp(*this); }
    Dim computeShape() override;
};

} // namespace tpm

#ifdef PET_HAVE_NNET
#include "perf_engine.h"
#include "membound.h"
#endif
