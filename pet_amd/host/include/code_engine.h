// Whole-graph execution (role of the reference's include/code_engine.h). The
// reference prints a CUDA program full of cuDNN / cuBLAS calls and TVM kernels
// (src/Graph/code_engine.cc:91-243). Here the graph becomes a single-GPU HIP
// graph runtime, in two forms:
//   * instantiate(): an in-process GraphExec whose operators' launches are
//     captured once on the backend stream and replayed with hipGraphLaunch;
//   * genCode(): a self-contained C++ program against pet_hip.h that allocates
//     the tensors, captures the same launches and prints "Time(ms)".
#pragma once
#include "graph.h"
#include "operator.h"
#include "perf_engine.h"
#include <string>

namespace tpm {

class GraphExec {
  public:
    ~GraphExec();
    // One replay of the captured graph, asynchronous on the backend stream.
    bool launch();
    bool sync();
    // Mean ms per replay (hipEvent bracket, like the emitted program's loop at
    // src/Graph/code_engine.cc:194-217: default 100 warm-up + 1000 timed).
    double time(int warmup = 100, int rounds = 1000);
    size_t numKernelOps() const { return nLaunchOps; }
    size_t numAliasedOps() const { return nAliasOps; }
    // Transposes that run as part of the transpose that follows them.
    size_t numFoldedOps() const { return nFoldedOps; }
    // output initialisations of accumulating contractions, batched into the first launch
    size_t numHoistedFills() const { return nHoistedFills; }

  private:
    friend class CodeEngine;
    pet_hip_graph_t graph = nullptr;
    size_t nLaunchOps = 0, nAliasOps = 0, nFoldedOps = 0, nHoistedFills = 0;
};

class CodeEngine {
  public:
    CodeEngine() {}
    void importPerfEngine(std::shared_ptr<PerfEngine> pe) { perfEngine = std::move(pe); }

    // Allocates every tensor on the device, makes split / concat on dim 0 and
    // reshape zero-copy aliases (as src/Graph/code_engine.cc:133-155, 1681-1690
    // do with pointer arithmetic), runs weight-only operators once, and
    // captures the remaining operators in topological order.
    std::unique_ptr<GraphExec> instantiate(std::shared_ptr<SubGraph> &graph);

    std::string genCode(std::shared_ptr<SubGraph> &graph);
    int genCode(std::shared_ptr<SubGraph> &graph, const std::string &filename);

  private:
    void importAlgos(const OpVec &order);
    std::shared_ptr<PerfEngine> perfEngine;
};

} // namespace tpm
