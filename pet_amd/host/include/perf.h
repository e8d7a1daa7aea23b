// Keys and results of the per-operator timing memo (role of the reference's
// include/perf.h). The cuDNN / cuBLAS algorithm enums of the reference
// (perf.h:27-69) become a plain int naming the kernel variant that was timed.
#pragma once
#include "common.h"
#include <tuple>

namespace tpm {

// n, c, h, w, f, r, s, ph, pw, sh, sw, dh, dw, g, bias, act
typedef std::tuple<int, int, int, int, int, int, int, int, int, int, int, int, int, int, int, int>
    ConvArgs;
// transA, transB, b, m, n, k
typedef std::tuple<bool, bool, int, int, int, int> MatmulArgs;
// kh, kw, ph, pw, sh, sw, dh, dw
typedef std::tuple<int, int, int, int, int, int, int, int> PoolArgs;

struct ConvResult {
    double time;          // ms per launch
    int algo;             // 0: the backend's own choice (one fused kernel)
    size_t workspaceSize; // always 0: the kernels need no workspace
    bool fuseAct;         // bias + activation are fused in the epilogue
};

struct ConvTransResult {
    double time;
    int algo; // one kernel: always 0
    size_t workspaceSize;
};

struct MatmulResult {
    double time;
    bool useStrideBatchAPI;
    int algo;
};

} // namespace tpm
