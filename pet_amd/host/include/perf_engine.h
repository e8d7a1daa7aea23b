// Per-operator timing context (role of the reference's include/perf_engine.h).
// The reference owns 4 x 1 GiB operand buffers plus a 7 GiB cuDNN workspace
// (src/Graph/perf_engine.cc:31-42) and cuDNN / cuBLAS handles; here the scratch
// operands are sized on demand (the kernels need no workspace), are filled once
// with uniform noise on the device, and the only handle is the backend stream.
#pragma once
#include "common.h"
#include "operator.h"
#include "perf.h"

namespace tpm {

class PerfEngine {
  public:
    PerfEngine();
    ~PerfEngine();
    PerfEngine(const PerfEngine &) = delete;

    void setPenalty(int flag) { penaltyFlag = flag; }
    int withPenalty() const { return penaltyFlag; }

    // Scratch operands of at least `elems` floats each, grown when needed.
    float *getInputPtr(size_t elems = 0) { return scratch(0, elems); }
    float *getWeightPtr(size_t elems = 0) { return scratch(1, elems); }
    float *getOutputPtr(size_t elems = 0) { return scratch(2, elems); }
    float *getBiasPtr(size_t elems = 0) { return scratch(3, elems); }
    float *getMatA(size_t elems = 0) { return scratch(0, elems); }
    float *getMatB(size_t elems = 0) { return scratch(1, elems); }
    float *getMatC(size_t elems = 0) { return scratch(2, elems); }
    float *getWorkspace() { return nullptr; } // no kernel here takes one
    pet_hip_stream_t stream() const { return petStream(); }

    int getConvAlgo(const ConvArgs &args) { return convPerf.at(args).algo; }
    int getMatmulAlgo(const MatmulArgs &args) { return matmulPerf.at(args).algo; }

    template <class OpArgs> double getOpPerf(Operator::OpType, const OpArgs &) { return 0.0; }
    double getOpPerf(Operator::OpType t, const ConvArgs &args) {
        return t == Operator::ConvTrans ? convTransPerf.at(args).time : convPerf.at(args).time;
    }
    double getOpPerf(Operator::OpType t, const G2BMMGBMMLArgs &args) {
        return (t == Operator::G2BMM ? g2bmmPerf : gbmmlPerf).at(args);
    }
    int getConvTransAlgo(const ConvArgs &args) { return convTransPerf.at(args).algo; }
    double getOpPerf(Operator::OpType, const MatmulArgs &args) { return matmulPerf.at(args).time; }
    double getOpPerf(Operator::OpType t, const PoolArgs &args) {
        return (t == Operator::MaxPool ? maxPoolPerf : avgPoolPerf).at(args);
    }

    template <class OpArgs> bool checkOpPerf(Operator::OpType, const OpArgs &) { return true; }
    bool checkOpPerf(Operator::OpType t, const ConvArgs &args) {
        return (t == Operator::ConvTrans ? convTransPerf.count(args) : convPerf.count(args)) != 0;
    }
    bool checkOpPerf(Operator::OpType t, const G2BMMGBMMLArgs &args) {
        return (t == Operator::G2BMM ? g2bmmPerf : gbmmlPerf).count(args) != 0;
    }
    bool checkOpPerf(Operator::OpType, const MatmulArgs &args) {
        return matmulPerf.count(args) != 0;
    }
    bool checkOpPerf(Operator::OpType t, const PoolArgs &args) {
        return (t == Operator::MaxPool ? maxPoolPerf : avgPoolPerf).count(args) != 0;
    }

    void saveOpPerf(uint32_t, const ConvArgs &args, const ConvResult &r) { convPerf[args] = r; }
    void saveOpPerf(uint32_t, const ConvArgs &args, const ConvTransResult &r) {
        convTransPerf[args] = r;
    }
    void saveOpPerf(uint32_t t, const G2BMMGBMMLArgs &args, float ms) {
        (t == Operator::G2BMM ? g2bmmPerf : gbmmlPerf)[args] = ms;
    }
    void saveOpPerf(uint32_t, const MatmulArgs &args, const MatmulResult &r) {
        matmulPerf[args] = r;
    }
    void saveOpPerf(uint32_t t, const PoolArgs &args, float ms) {
        (t == Operator::MaxPool ? maxPoolPerf : avgPoolPerf)[args] = ms;
    }

    // Measured copy bandwidth of this GPU in GiB/s (a large view-copy launch),
    // used where the reference hard-codes 200 GiB/s for layout operators
    // (src/Graph/operator.cc:2390).
    double layoutBandwidthGiBs();

    void dumpPerfData();

  private:
    float *scratch(int which, size_t elems);

    int penaltyFlag = 1;
    std::map<ConvArgs, ConvResult> convPerf;
    std::map<ConvArgs, ConvTransResult> convTransPerf;
    std::map<MatmulArgs, MatmulResult> matmulPerf;
    std::map<G2BMMGBMMLArgs, float> g2bmmPerf, gbmmlPerf;
    std::map<PoolArgs, float> maxPoolPerf, avgPoolPerf;
    float *buf[4] = {nullptr, nullptr, nullptr, nullptr};
    size_t bufElems[4] = {0, 0, 0, 0};
    double bandwidth = 0.0;
};

} // namespace tpm
