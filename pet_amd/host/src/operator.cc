#include "operator.h"
#include "perf_engine.h"

#include <algorithm>
#include <stdexcept>
#include <string>

namespace tpm {

// The constructors assert the validity of their operands, as the reference's do. A front end
// that builds operators from a file it does not control (Graph::importOnnx) asks for an
// exception instead for the duration of its work.
thread_local int invalidOperandsThrow = 0;
InvalidOperandsThrow::InvalidOperandsThrow() { ++invalidOperandsThrow; }
InvalidOperandsThrow::~InvalidOperandsThrow() { --invalidOperandsThrow; }
#define PET_OPERANDS_VALID(cond)                                                               \
    do {                                                                                       \
        if (!(cond)) {                                                                         \
            if (invalidOperandsThrow)                                                          \
                throw std::invalid_argument(std::string(__func__) + ": operands it rejects");  \
            assert(cond);                                                                      \
        }                                                                                      \
    } while (0)

// ---- Operator base ------------------------------------------------------------

std::string Operator::getOpName(OpType t) {
    static const std::map<int, const char *> names = {
        {Unknown, "Unknown"},   {Conv, "Conv"},         {Matmul, "Matmul"},
        {ConvTrans, "ConvTrans"}, {G2BMM, "G2BMM"},     {GBMML, "GBMML"},
        {Pad, "Pad"},           {Slice, "Slice"},       {Concat, "Concat"},
        {Split, "Split"},       {Transpose, "Transpose"}, {Extend, "Extend"},
        {MaxPool, "MaxPool"},   {AvgPool, "AvgPool"},   {Add, "Add"},
        {Sub, "Sub"},           {Mul, "Mul"},           {Div, "Div"},
        {Pow, "Pow"},           {Gather, "Gather"},     {ReduceMean, "ReduceMean"},
        {Reshape, "Reshape"},   {Identity, "Identity"}, {BatchNorm, "BatchNorm"},
        {Softmax, "Softmax"},   {Activation, "Activation"}, {Resize, "Resize"},
        {MemBound, "MemBound"}, {Conv3d, "Conv3d"},     {LayerNorm, "LayerNorm"}};
    auto it = names.find(t);
    return it == names.end() ? "Unknown" : it->second;
}

bool Operator::allocOutputs() {
    for (auto t : outputs)
        if (!t->isValid() || !t->dataMalloc())
            return false;
    return true;
}

Tensor *Operator::compute() {
    if (outputs.empty())
        return nullptr;
    bool done = true;
    for (auto t : outputs)
        done = done && t->isComputed();
    if (done)
        return outputs[0];
    for (auto t : inputs)
        if (t == nullptr || !t->isValid()) {
            if (hostTrace())
                std::fprintf(stderr, "[pet] %s: invalid input\n", toString().c_str());
            return nullptr;
        }
    if (!allocOutputs()) {
        if (hostTrace())
            std::fprintf(stderr, "[pet] %s: output allocation failed\n", toString().c_str());
        return nullptr;
    }
    int status = launch(petStream());
    if (status != PET_HIP_OK) {
        if (hostTrace())
            std::fprintf(stderr, "[pet] %s: launch status %d: %s\n", toString().c_str(), status,
                         pet_hip_last_error());
        return nullptr;
    }
    for (auto t : outputs) {
        t->deviceWritten();
        t->setComputed();
        t->refreshHostMirrorInPlace();
    }
    return outputs[0];
}

int Operator::launchFused(pet_hip_stream_t, const float *, ActType, float *, unsigned) {
    return PET_HIP_ERR_UNSUPPORTED;
}

std::pair<std::vector<DimRange>, std::function<bool()>> Operator::compute(DimRange dr) {
    if (dr.notValid())
        return {};
    if (dr.isEmpty())
        return {std::vector<DimRange>(inputs.size(), DimRange::getEmpty()), []() { return true; }};
    return {std::vector<DimRange>(inputs.size(), DimRange::getAllPos()),
            [this]() { return compute() != nullptr; }};
}

bool Operator::computeShape(const TensorVec &ins, const TensorVec &outs) {
    if ((type != Concat && type != Add && type != Mul && ins.size() != (size_t)numInputs()) ||
        (type != Split && outs.size() != (size_t)numOutputs()))
        return false;
    for (auto t : ins)
        if (t == nullptr)
            return false;
    for (auto t : outs)
        if (t == nullptr)
            return false;
    if (!checkValid(ins))
        return false;
    inputs = ins;
    outputs = outs;
    Dim dm = computeShape();
    for (auto t : outputs)
        if (!t->isValid())
            return false;
    outputs[0]->setDims(dm);
    return true;
}

void Operator::inferSplittingPoints() {
    for (auto t : outputs)
        t->initSplittingPoints();
}

void Operator::getOptypeAttr(std::string &optype, std::map<std::string, std::string> &attr,
                             std::map<std::string, std::vector<int>> &) const {
    optype = getOpName(type);
    attr.clear();
}

double Operator::timeLaunches(int rounds, int warmupRounds) {
    if (!petInit())
        return INFINITY;
    for (auto t : inputs)
        if (!t->devicePtr())
            return INFINITY;
    if (!allocOutputs())
        return INFINITY;
    pet_hip_stream_t s = petStream();
    for (int i = 0; i < warmupRounds; ++i)
        if (launch(s) != PET_HIP_OK)
            return INFINITY;
    pet_hip_event_t e0 = nullptr, e1 = nullptr;
    pet_hip_event_create(&e0);
    pet_hip_event_create(&e1);
    pet_hip_event_record(e0, s);
    for (int i = 0; i < rounds; ++i)
        launch(s);
    pet_hip_event_record(e1, s);
    pet_hip_event_sync(e1);
    float ms = 0.f;
    pet_hip_event_elapsed_ms(&ms, e0, e1);
    pet_hip_event_destroy(e0);
    pet_hip_event_destroy(e1);
    return rounds > 0 ? (double)ms / rounds : 0.0;
}

namespace {

// Times `fn` (a launch on the backend stream) with an event bracket.
template <class F> double timeFn(F fn, int rounds, int warmupRounds) {
    pet_hip_stream_t s = petStream();
    for (int i = 0; i < warmupRounds; ++i)
        if (fn(s) != PET_HIP_OK)
            return INFINITY;
    pet_hip_event_t e0 = nullptr, e1 = nullptr;
    pet_hip_event_create(&e0);
    pet_hip_event_create(&e1);
    pet_hip_event_record(e0, s);
    for (int i = 0; i < rounds; ++i)
        fn(s);
    pet_hip_event_record(e1, s);
    pet_hip_event_sync(e1);
    float ms = 0.f;
    pet_hip_event_elapsed_ms(&ms, e0, e1);
    pet_hip_event_destroy(e0);
    pet_hip_event_destroy(e1);
    return rounds > 0 ? (double)ms / rounds : 0.0;
}

uint64_t hashDims(uint64_t h, const Dim &d) {
    h = hashAppend(h, d.size());
    for (int v : d)
        h = hashAppend(h, (uint64_t)(int64_t)v);
    return h;
}

std::string tensorTag(const char *name, const Tensor *t) {
    return std::string(name) + "=" + std::to_string(t->getHash());
}

} // namespace

// ---- ConvOp ---------------------------------------------------------------------

ConvOp::ConvOp(Tensor *input, Tensor *weight, Tensor *output, int ph, int pw, int sh, int sw,
               int dh, int dw, Tensor *bias, ActType act)
    : Operator(Conv, {input, weight}, {output}), ph(ph), pw(pw), sh(sh), sw(sw), dh(dh), dw(dw),
      bias(bias), act(act), padding(Other) {
    weight->setType(Tensor::Weight);
    PET_OPERANDS_VALID(checkValid({input, weight}));
    computeShape();
    setPaddingMode();
    initHash();
}

ConvOp::ConvOp(Tensor *input, Tensor *weight, int ph, int pw, int sh, int sw, int dh, int dw,
               Tensor *bias, ActType act)
    : ConvOp(input, weight, new Tensor(), ph, pw, sh, sw, dh, dw, bias, act) {}

ConvOp::ConvOp(int ph, int pw, int sh, int sw, int dh, int dw, Tensor *bias, ActType act)
    : Operator(Conv), ph(ph), pw(pw), sh(sh), sw(sw), dh(dh), dw(dw), bias(bias), act(act),
      padding(Other) {
    initHash();
}

ConvOp::ConvOp(Tensor *input, Tensor *weight, Tensor *output, PaddingMode pm, int sh, int sw,
               int dh, int dw, Tensor *bias, ActType act)
    : Operator(Conv, {input, weight}, {output}), sh(sh), sw(sw), dh(dh), dw(dw), bias(bias),
      act(act), padding(pm) {
    assert(pm != Other);
    weight->setType(Tensor::Weight);
    PET_OPERANDS_VALID(checkValid({input, weight}));
    computeShape();
    initHash();
}

ConvOp::ConvOp(Tensor *input, Tensor *weight, PaddingMode pm, int sh, int sw, int dh, int dw,
               Tensor *bias, ActType act)
    : ConvOp(input, weight, new Tensor(), pm, sh, sw, dh, dw, bias, act) {}

ConvOp::ConvOp(PaddingMode pm, int sh, int sw, int dh, int dw, Tensor *bias, ActType act)
    : Operator(Conv), sh(sh), sw(sw), dh(dh), dw(dw), bias(bias), act(act), padding(pm) {
    initHash();
}

ConvOp::ConvOp(const ConvOp &rhs)
    : Operator(rhs), ph(rhs.ph), pw(rhs.pw), sh(rhs.sh), sw(rhs.sw), dh(rhs.dh), dw(rhs.dw),
      bias(rhs.bias), act(rhs.act), padding(rhs.padding), algo(rhs.algo) {}

void ConvOp::initHash() {
    hash = type;
    hash = hashAppend(hash, padding);
    if (padding == Other) {
        hash = hashAppend(hash, ph);
        hash = hashAppend(hash, pw);
    }
    for (int v : {sh, sw, dh, dw})
        hash = hashAppend(hash, v);
    hash = hashPack(hash);
}

// Shape rules of the reference (src/Graph/operator.cc:219-231): with explicit
// padding o = (i - (k - s) d + 2p) / s; Same: o = i / s and the padding that
// gives it; Valid: no padding.
void ConvOp::outputExtent(int h, int w, int r, int s, int &oh, int &ow) {
    if (padding == Same) {
        oh = h / sh;
        ow = w / sw;
        ph = (h - oh * sh + (r - sh) * dh) / 2;
        pw = (w - ow * sw + (s - sw) * dw) / 2;
        return;
    }
    if (padding == Valid)
        ph = pw = 0;
    oh = pet_hip_conv_out_dim(h, r, ph, sh, dh);
    ow = pet_hip_conv_out_dim(w, s, pw, sw, dw);
}

Dim ConvOp::computeShape() {
    auto in = inputs[0]->getDims(), wt = inputs[1]->getDims();
    int oh, ow;
    outputExtent(in[2], in[3], wt[2], wt[3], oh, ow);
    Dim ret = {in[0], wt[0], oh, ow};
    outputs[0]->setDims(ret);
    outputs[0]->setType(Tensor::Input);
    return ret;
}

Dim ConvOp::computeOutputPenalty(const Dim &p) {
    assert(p.size() == 4);
    auto in = inputs[0]->getDims(), wt = inputs[1]->getDims();
    int oh, ow;
    outputExtent(in[2] + p[2], in[3] + p[3], wt[2], wt[3], oh, ow);
    auto out = outputs[0]->getDims();
    return {in[0] + p[0] - out[0], 0, oh - out[2], ow - out[3]};
}

void ConvOp::setPaddingMode() {
    auto in = inputs[0]->getDims(), out = outputs[0]->getDims();
    if (in[2] == out[2] && in[3] == out[3])
        padding = Same;
    else if (ph == 0 && pw == 0)
        padding = Valid;
}

bool ConvOp::checkValid(const TensorVec &ins) {
    auto input = ins[0], weight = ins[1];
    if (input->getType() != Tensor::Input || weight->getType() != Tensor::Weight)
        return false;
    if (input->getDims().size() != 4 || weight->getDims().size() != 4)
        return false;
    return weight->getDims()[1] > 0 && input->getDims()[1] % weight->getDims()[1] == 0;
}

ConvArgs ConvOp::getArgs(int withPenalty) const {
    auto in = inputs[0]->getDims();
    auto pen = static_cast<const Tensor *>(inputs[0])->getPenalty();
    auto wt = inputs[1]->getDims();
    int n = in[0] + withPenalty * pen[0], c = in[1] + withPenalty * pen[1];
    int h = in[2] + withPenalty * pen[2], w = in[3] + withPenalty * pen[3];
    return ConvArgs{n, c, h, w, wt[0], wt[2], wt[3], ph, pw, sh, sw, dh, dw, c / wt[1],
                    bias ? 1 : 0, (int)act};
}

int ConvOp::launch(pet_hip_stream_t stream) {
    auto in = inputs[0]->getDims(), wt = inputs[1]->getDims();
    int groups = in[1] / wt[1];
    // the reference's compute() returns nullptr when f % g != 0
    if (groups <= 0 || wt[0] % groups != 0)
        return PET_HIP_ERR_INVALID;
    if (algo != 0)
        return pet_hip_conv2d_ex_f32(inputs[0]->devicePtr(), inputs[1]->devicePtr(),
                                     bias ? bias->devicePtr() : nullptr, nullptr,
                                     outputs[0]->devicePtr(), in[0], in[1], in[2], in[3], wt[0],
                                     wt[2], wt[3], ph, pw, sh, sw, dh, dw, groups, (int)act,
                                     PET_HIP_CONV_ALGO(algo), stream);
    return pet_hip_conv2d_f32(inputs[0]->devicePtr(), inputs[1]->devicePtr(),
                              bias ? bias->devicePtr() : nullptr, outputs[0]->devicePtr(), in[0],
                              in[1], in[2], in[3], wt[0], wt[2], wt[3], ph, pw, sh, sw, dh, dw,
                              groups, (int)act, stream);
}

int ConvOp::launchFused(pet_hip_stream_t stream, const float *residual, ActType finalAct,
                        float *out, unsigned flags) {
    auto in = inputs[0]->getDims(), wt = inputs[1]->getDims();
    int groups = in[1] / wt[1];
    if (groups <= 0 || wt[0] % groups != 0 || (residual != nullptr && act != None))
        return PET_HIP_ERR_INVALID;
    return pet_hip_conv2d_ex_f32(inputs[0]->devicePtr(), inputs[1]->devicePtr(),
                                 bias ? bias->devicePtr() : nullptr, residual, out, in[0], in[1],
                                 in[2], in[3], wt[0], wt[2], wt[3], ph, pw, sh, sw, dh, dw, groups,
                                 (int)finalAct, flags | PET_HIP_CONV_ALGO(algo), stream);
}

int ConvOp::launchView(pet_hip_stream_t stream, const float *x, const pet_hip_conv_view *xView,
                       float *y, const pet_hip_conv_view *yView, unsigned flags) {
    auto in = inputs[0]->getDims(), wt = inputs[1]->getDims();
    int groups = in[1] / wt[1];
    if (groups <= 0 || wt[0] % groups != 0)
        return PET_HIP_ERR_INVALID;
    return pet_hip_conv2d_view_f32(x, xView, inputs[1]->devicePtr(),
                                   bias ? bias->devicePtr() : nullptr, nullptr, y, yView, in[0],
                                   in[1], in[2], in[3], wt[0], wt[2], wt[3], ph, pw, sh, sw, dh, dw,
                                   groups, (int)act, flags | PET_HIP_CONV_ALGO(algo), stream);
}

bool ConvOp::accumulates() const {
    auto in = inputs[0]->getDims(), wt = inputs[1]->getDims();
    int groups = wt[1] > 0 ? in[1] / wt[1] : 0, yes = 0;
    if (groups <= 0)
        return false;
    return pet_hip_conv2d_accumulates(in[0], in[1], in[2], in[3], wt[0], wt[2], wt[3], ph, pw, sh,
                                      sw, dh, dw, groups, &yes) == PET_HIP_OK &&
           yes != 0;
}

double ConvOp::perf(PerfEngine *pe, int rounds, int warmupRounds) {
    ConvArgs args = getArgs(pe->withPenalty());
    if (pe->checkOpPerf(Conv, args)) {
        algo = pe->getConvAlgo(args);
        return pe->getOpPerf(Conv, args);
    }
    int n, c, h, w, f, r, s, ph_, pw_, sh_, sw_, dh_, dw_, g, bi, ac;
    std::tie(n, c, h, w, f, r, s, ph_, pw_, sh_, sw_, dh_, dw_, g, bi, ac) = args;
    ConvResult best{INFINITY, 0, 0, true};
    if (g > 0 && c % g == 0 && f % g == 0) {
        int oh = pet_hip_conv_out_dim(h, r, ph_, sh_, dh_);
        int ow = pet_hip_conv_out_dim(w, s, pw_, sw_, dw_);
        if (oh > 0 && ow > 0) {
            float *x = pe->getInputPtr((size_t)n * c * h * w);
            float *wt = pe->getWeightPtr((size_t)f * (c / g) * r * s);
            float *y = pe->getOutputPtr((size_t)n * f * oh * ow);
            float *b = pe->getBiasPtr((size_t)f);
            if (x && wt && y && b) {
                // Bias and activation ride in the kernel's epilogue; what there is to choose
                // is how the K loop is shared out (the reference loops over cuDNN's
                // algorithms here, src/Graph/operator.cc:352-470). The cost model's choice
                // is timed in full; another algorithm has to beat it by 3 % on a shorter
                // run, then confirm on a full one, to be taken.
                auto run = [&](int a, int rds, int warm) {
                    return timeFn(
                        [&](pet_hip_stream_t st) {
                            return pet_hip_conv2d_ex_f32(x, wt, b, nullptr, y, n, c, h, w, f, r, s,
                                                         ph_, pw_, sh_, sw_, dh_, dw_, g, ac,
                                                         PET_HIP_CONV_ALGO(a), st);
                        },
                        rds, warm);
                };
                best.time = run(0, rounds, warmupRounds);
                static const bool tune = getenv("PET_HOST_NO_ALGO_SEARCH") == nullptr;
                const int quick = std::max(10, rounds / 4);
                for (int a = 1; tune && a < PET_HIP_CONV_ALGO_COUNT; ++a) {
                    double t = run(a, quick, std::min(warmupRounds, 10));
                    if (!(t < 0.97 * best.time))
                        continue;
                    t = run(a, rounds, std::min(warmupRounds, 20));
                    if (t < 0.97 * best.time) {
                        best.time = t;
                        best.algo = a;
                    }
                }
            }
        }
    }
    pe->saveOpPerf(Conv, args, best);
    algo = best.algo;
    return best.time;
}

bool ConvOp::same(const ConvOp &rhs) {
    bool ret = padding == Other ? (ph == rhs.ph && pw == rhs.pw) : padding == rhs.padding;
    return ret && sh == rhs.sh && sw == rhs.sw && dh == rhs.dh && dw == rhs.dw;
}

std::string ConvOp::toString() const {
    std::ostringstream os;
    os << "Conv[" << hash << "](";
    if (inputs.size() == 2)
        os << dimToString(inputs[0]->getDims()) << "," << dimToString(inputs[1]->getDims()) << ",";
    os << "p=[" << ph << "," << pw << "],s=[" << sh << "," << sw << "],d=[" << dh << "," << dw
       << "],act=" << act;
    if (inputs.size() == 2)
        os << "," << tensorTag("input", inputs[0]) << "," << tensorTag("weight", inputs[1]) << ","
           << tensorTag("output", outputs[0]);
    os << ")";
    return os.str();
}

// ---- ConvTransOp ----------------------------------------------------------------

ConvTransOp::ConvTransOp(Tensor *input, Tensor *weight, Tensor *output, int ph, int pw, int sh,
                         int sw, int dh, int dw, int oph, int opw, Tensor *bias, ActType act)
    : Operator(ConvTrans, {input, weight}, {output}), ph(ph), pw(pw), sh(sh), sw(sw), dh(dh),
      dw(dw), oph(oph), opw(opw), bias(bias), act(act), padding(Other) {
    weight->setType(Tensor::Weight);
    PET_OPERANDS_VALID(checkValid({input, weight}));
    computeShape();
    setPaddingMode();
    initHash();
}

ConvTransOp::ConvTransOp(Tensor *input, Tensor *weight, int ph, int pw, int sh, int sw, int dh,
                         int dw, int oph, int opw, Tensor *bias, ActType act)
    : ConvTransOp(input, weight, new Tensor(), ph, pw, sh, sw, dh, dw, oph, opw, bias, act) {}

ConvTransOp::ConvTransOp(int ph, int pw, int sh, int sw, int dh, int dw, int oph, int opw,
                         Tensor *bias, ActType act)
    : Operator(ConvTrans), ph(ph), pw(pw), sh(sh), sw(sw), dh(dh), dw(dw), oph(oph), opw(opw),
      bias(bias), act(act), padding(Other) {
    initHash();
}

// The padding-mode constructors keep the mode for hashing and same(); the reference never
// derives a padding size from it for this operator (its computeShape reads ph and pw as
// they are, src/Graph/operator.cc:1055-1072), so they stay 0 here as well.
ConvTransOp::ConvTransOp(Tensor *input, Tensor *weight, Tensor *output, PaddingMode pm, int sh,
                         int sw, int dh, int dw, int oph, int opw, Tensor *bias, ActType act)
    : Operator(ConvTrans, {input, weight}, {output}), sh(sh), sw(sw), dh(dh), dw(dw), oph(oph),
      opw(opw), bias(bias), act(act), padding(pm) {
    weight->setType(Tensor::Weight);
    PET_OPERANDS_VALID(checkValid({input, weight}));
    computeShape();
    initHash();
}

ConvTransOp::ConvTransOp(Tensor *input, Tensor *weight, PaddingMode pm, int sh, int sw, int dh,
                         int dw, int oph, int opw, Tensor *bias, ActType act)
    : ConvTransOp(input, weight, new Tensor(), pm, sh, sw, dh, dw, oph, opw, bias, act) {}

ConvTransOp::ConvTransOp(PaddingMode pm, int sh, int sw, int dh, int dw, int oph, int opw,
                         Tensor *bias, ActType act)
    : Operator(ConvTrans), sh(sh), sw(sw), dh(dh), dw(dw), oph(oph), opw(opw), bias(bias),
      act(act), padding(pm) {
    initHash();
}

ConvTransOp::ConvTransOp(const ConvTransOp &rhs)
    : Operator(rhs), ph(rhs.ph), pw(rhs.pw), sh(rhs.sh), sw(rhs.sw), dh(rhs.dh), dw(rhs.dw),
      oph(rhs.oph), opw(rhs.opw), bias(rhs.bias), act(rhs.act), padding(rhs.padding) {}

void ConvTransOp::initHash() {
    hash = type;
    hash = hashAppend(hash, padding);
    if (padding == Other) {
        hash = hashAppend(hash, ph);
        hash = hashAppend(hash, pw);
    }
    for (int v : {sh, sw, dh, dw, oph, opw})
        hash = hashAppend(hash, v);
    hash = hashPack(hash);
}

// input [n,h,w,f], weight [r,s,f,c] -> [n, oh, ow, c] (src/Graph/operator.cc:1055-1072)
Dim ConvTransOp::computeShape() {
    auto in = inputs[0]->getDims(), wt = inputs[1]->getDims();
    Dim ret = {in[0], pet_hip_conv_trans_out_dim(in[1], wt[0], ph, sh, dh, oph),
               pet_hip_conv_trans_out_dim(in[2], wt[1], pw, sw, dw, opw), wt[3]};
    outputs[0]->setDims(ret);
    outputs[0]->setType(Tensor::Input);
    return ret;
}

void ConvTransOp::setPaddingMode() {
    auto in = inputs[0]->getDims(), out = outputs[0]->getDims();
    if (in[1] == out[1] && in[2] == out[2])
        padding = Same;
    else if (ph == 0 && pw == 0)
        padding = Valid;
}

bool ConvTransOp::checkValid(const TensorVec &ins) {
    auto input = ins[0], weight = ins[1];
    if (input->getType() != Tensor::Input || weight->getType() != Tensor::Weight)
        return false;
    if (input->getDims().size() != 4 || weight->getDims().size() != 4)
        return false;
    // grouped and dilated forms are asserted away upstream (src/Graph/operator.cc:1098-1101)
    return input->getDims()[3] == weight->getDims()[2];
}

ConvArgs ConvTransOp::getArgs(int withPenalty) const {
    auto in = inputs[0]->getDims();
    auto pen = static_cast<const Tensor *>(inputs[0])->getPenalty();
    auto wt = inputs[1]->getDims();
    int n = in[0] + withPenalty * pen[0], h = in[1] + withPenalty * pen[1];
    int w = in[2] + withPenalty * pen[2], f = in[3] + withPenalty * pen[3];
    return ConvArgs{n, wt[3], h, w, f, wt[0], wt[1], ph, pw, sh, sw, dh, dw, 1, bias ? 1 : 0,
                    (int)act};
}

int ConvTransOp::launch(pet_hip_stream_t stream) {
    auto in = inputs[0]->getDims(), wt = inputs[1]->getDims();
    return pet_hip_conv_trans_f32(inputs[0]->devicePtr(), inputs[1]->devicePtr(),
                                  bias ? bias->devicePtr() : nullptr, outputs[0]->devicePtr(),
                                  in[0], in[1], in[2], in[3], wt[0], wt[1], wt[3], ph, pw, sh, sw,
                                  dh, dw, oph, opw, (int)act, stream);
}

// One kernel: nothing to choose between, where the reference loops over cuDNN's
// backward-data algorithms (src/Graph/operator.cc:1113-1287). The memo key has no output
// padding, as upstream (include/operator.h:597), so neither do the timed launches.
double ConvTransOp::perf(PerfEngine *pe, int rounds, int warmupRounds) {
    ConvArgs args = getArgs(pe->withPenalty());
    if (pe->checkOpPerf(ConvTrans, args))
        return pe->getOpPerf(ConvTrans, args);
    int n, c, h, w, f, r, s, ph_, pw_, sh_, sw_, dh_, dw_, g, bi, ac;
    std::tie(n, c, h, w, f, r, s, ph_, pw_, sh_, sw_, dh_, dw_, g, bi, ac) = args;
    ConvTransResult res{INFINITY, 0, 0};
    const int oh = pet_hip_conv_trans_out_dim(h, r, ph_, sh_, dh_, 0);
    const int ow = pet_hip_conv_trans_out_dim(w, s, pw_, sw_, dw_, 0);
    if (oh > 0 && ow > 0) {
        float *x = pe->getInputPtr((size_t)n * h * w * f);
        float *wt = pe->getWeightPtr((size_t)r * s * f * c);
        float *y = pe->getOutputPtr((size_t)n * oh * ow * c);
        float *b = pe->getBiasPtr((size_t)c);
        if (x && wt && y && b)
            res.time = timeFn(
                [&](pet_hip_stream_t st) {
                    return pet_hip_conv_trans_f32(x, wt, bi ? b : nullptr, y, n, h, w, f, r, s, c,
                                                  ph_, pw_, sh_, sw_, dh_, dw_, 0, 0, ac, st);
                },
                rounds, warmupRounds);
    }
    pe->saveOpPerf(ConvTrans, args, res);
    return res.time;
}

bool ConvTransOp::same(const ConvTransOp &rhs) {
    bool ret = padding == Other ? (ph == rhs.ph && pw == rhs.pw) : padding == rhs.padding;
    return ret && sh == rhs.sh && sw == rhs.sw && dh == rhs.dh && dw == rhs.dw;
}

std::string ConvTransOp::toString() const {
    std::ostringstream os;
    os << "ConvTrans[" << hash << "](";
    if (inputs.size() == 2)
        os << dimToString(inputs[0]->getDims()) << "," << dimToString(inputs[1]->getDims()) << ",";
    os << "p=[" << ph << "," << pw << "],s=[" << sh << "," << sw << "],d=[" << dh << "," << dw
       << "],op=[" << oph << ", " << opw << "],act=" << act;
    if (inputs.size() == 2)
        os << "," << tensorTag("input", inputs[0]) << "," << tensorTag("weight", inputs[1]) << ","
           << tensorTag("output", outputs[0]);
    os << ")";
    return os.str();
}

// ---- Conv3dOp -------------------------------------------------------------------

Conv3dOp::Conv3dOp(Tensor *input, Tensor *weight, Tensor *output, const Dim &pad,
                   const Dim &stride, const Dim &dilation, Tensor *bias, ActType act)
    : Operator(Conv3d, {input, weight}, {output}), pad(pad), stride(stride), dilation(dilation),
      bias(bias), act(act) {
    weight->setType(Tensor::Weight);
    PET_OPERANDS_VALID(checkValid({input, weight}));
    computeShape();
    initHash();
}

Conv3dOp::Conv3dOp(const Conv3dOp &rhs)
    : Operator(rhs), pad(rhs.pad), stride(rhs.stride), dilation(rhs.dilation), bias(rhs.bias),
      act(rhs.act), algo(rhs.algo) {}

Conv3dOp::~Conv3dOp() {
    if (packed)
        pet_hip_free(packed);
}

bool Conv3dOp::usesPackedFilters() const {
    return packed != nullptr && packedElems == inputs[1]->size() &&
           packedVersion == inputs[1]->dataVersion();
}

bool Conv3dOp::prepackFilters(pet_hip_stream_t stream) {
    Tensor *w = inputs[1];
    const Dim &wt = w->getDims();
    const float *src = w->devicePtr(); // settles the upload, and with it the version
    if (src == nullptr)
        return false;
    if (packed == nullptr || packedElems != w->size()) {
        if (packed)
            pet_hip_free(packed);
        packed = nullptr;
        void *buf = nullptr;
        if (pet_hip_malloc(&buf, w->size() * sizeof(float)) != PET_HIP_OK)
            return false;
        packed = (float *)buf;
        packedElems = w->size();
    }
    int rc = pet_hip_conv3d_pack_filters(src, packed, wt[0], wt[1], wt[2], wt[3], wt[4], stream);
    if (rc != PET_HIP_OK) { // PET_HIP_ERR_UNSUPPORTED: this shape keeps its layout
        pet_hip_free(packed);
        packed = nullptr;
        packedElems = 0;
        return false;
    }
    packedVersion = w->dataVersion();
    return true;
}

void Conv3dOp::initHash() {
    hash = type;
    hash = hashDims(hashDims(hashDims(hash, pad), stride), dilation);
    hash = hashPack(hash);
}

bool Conv3dOp::checkValid(const TensorVec &ins) {
    if (ins[0]->getDims().size() != 5 || ins[1]->getDims().size() != 5)
        return false;
    if (pad.size() != 3 || stride.size() != 3 || dilation.size() != 3)
        return false;
    return ins[1]->getDims()[1] > 0 && ins[0]->getDims()[1] % ins[1]->getDims()[1] == 0;
}

Dim Conv3dOp::computeShape() {
    auto in = inputs[0]->getDims(), wt = inputs[1]->getDims();
    Dim ret = {in[0], wt[0], 0, 0, 0};
    for (int a = 0; a < 3; ++a)
        ret[2 + a] = pet_hip_conv_out_dim(in[2 + a], wt[2 + a], pad[a], stride[a], dilation[a]);
    outputs[0]->setDims(ret);
    outputs[0]->setType(Tensor::Input);
    return ret;
}

int Conv3dOp::launch(pet_hip_stream_t stream) {
    auto in = inputs[0]->getDims(), wt = inputs[1]->getDims();
    int groups = in[1] / wt[1];
    if (groups <= 0 || wt[0] % groups != 0)
        return PET_HIP_ERR_INVALID;
    if (algo != 0)
        return launchFused(stream, nullptr, act, outputs[0]->devicePtr(), 0);
    const float *w = inputs[1]->devicePtr();
    auto entry = pet_hip_conv3d_f32;
    if (usesPackedFilters()) {
        w = packed;
        entry = pet_hip_conv3d_packed_f32;
    }
    return entry(inputs[0]->devicePtr(), w, bias ? bias->devicePtr() : nullptr,
                 outputs[0]->devicePtr(), in[0], in[1], in[2], in[3], in[4], wt[0], wt[2], wt[3],
                 wt[4], pad[0], pad[1], pad[2], stride[0], stride[1], stride[2], dilation[0],
                 dilation[1], dilation[2], groups, (int)act, stream);
}

int Conv3dOp::launchFused(pet_hip_stream_t stream, const float *residual, ActType finalAct,
                          float *out, unsigned flags) {
    auto in = inputs[0]->getDims(), wt = inputs[1]->getDims();
    int groups = in[1] / wt[1];
    if (groups <= 0 || wt[0] % groups != 0 || (residual != nullptr && act != None))
        return PET_HIP_ERR_INVALID;
    const bool usePacked = usesPackedFilters();
    return pet_hip_conv3d_ex_f32(inputs[0]->devicePtr(), usePacked ? packed : inputs[1]->devicePtr(),
                                 usePacked, bias ? bias->devicePtr() : nullptr, residual, out,
                                 in[0], in[1], in[2], in[3], in[4], wt[0], wt[2], wt[3], wt[4],
                                 pad[0], pad[1], pad[2], stride[0], stride[1], stride[2],
                                 dilation[0], dilation[1], dilation[2], groups, (int)finalAct,
                                 flags | PET_HIP_CONV_ALGO(algo), stream);
}

bool Conv3dOp::accumulates() const {
    auto in = inputs[0]->getDims(), wt = inputs[1]->getDims();
    int groups = wt[1] > 0 ? in[1] / wt[1] : 0, yes = 0;
    if (groups <= 0)
        return false;
    return pet_hip_conv3d_accumulates(in[0], in[1], in[2], in[3], in[4], wt[0], wt[2], wt[3],
                                      wt[4], pad[0], pad[1], pad[2], stride[0], stride[1],
                                      stride[2], dilation[0], dilation[1], dilation[2], groups,
                                      usesPackedFilters(), &yes) == PET_HIP_OK &&
           yes != 0;
}

// The same search as ConvOp::perf, on the operator's own tensors (there is no memo for
// 3-D arguments: the reference has no such operator).
double Conv3dOp::perf(PerfEngine *, int rounds, int warmupRounds) {
    algo = 0;
    // time what the graph runtime will run: constant filters in their kt-major copy
    if (petInit() && inputs[1]->getType() == Tensor::Weight && inputs[1]->devicePtr())
        prepackFilters(petStream());
    double best = timeLaunches(rounds, warmupRounds);
    static const bool tune = getenv("PET_HOST_NO_ALGO_SEARCH") == nullptr;
    int bestAlgo = 0;
    const int quick = std::max(10, rounds / 4);
    for (int a = 1; tune && std::isfinite(best) && a < PET_HIP_CONV_ALGO_COUNT; ++a) {
        algo = a;
        double t = timeLaunches(quick, std::min(warmupRounds, 10));
        if (!(t < 0.97 * best))
            continue;
        t = timeLaunches(rounds, std::min(warmupRounds, 20));
        if (t < 0.97 * best) {
            best = t;
            bestAlgo = a;
        }
    }
    algo = bestAlgo;
    return best;
}

std::string Conv3dOp::toString() const {
    std::ostringstream os;
    os << "Conv3d[" << hash << "](" << dimToString(inputs[0]->getDims()) << ","
       << dimToString(inputs[1]->getDims()) << ",p=" << dimToString(pad)
       << ",s=" << dimToString(stride) << ",d=" << dimToString(dilation) << ",act=" << act << ")";
    return os.str();
}

// ---- MatmulOp -------------------------------------------------------------------

MatmulOp::MatmulOp(Tensor *A, Tensor *B, Tensor *C, bool transA, bool transB, Tensor *bias,
                   ActType act)
    : Operator(Matmul, {A, B}, {C}), transA(transA), transB(transB), bias(bias), act(act) {
    dimExtend(A);
    dimExtend(B);
    dimExtend(C);
    markWeight(A, B);
    PET_OPERANDS_VALID(checkValid({A, B}));
    if (C->getDims().empty())
        computeShape();
    initHash();
}

MatmulOp::MatmulOp(Tensor *A, Tensor *B, bool transA, bool transB, Tensor *bias, ActType act)
    : MatmulOp(A, B, new Tensor(), transA, transB, bias, act) {
    computeShape();
}

MatmulOp::MatmulOp(bool transA, bool transB, Tensor *bias, ActType act)
    : Operator(Matmul), transA(transA), transB(transB), bias(bias), act(act) {
    initHash();
}

void MatmulOp::initHash() {
    hash = type;
    hash = hashAppend(hash, transA);
    hash = hashAppend(hash, transB);
    hash = hashPack(hash);
}

// With two activations as operands the second is treated as the weight side
// (src/Graph/operator.cc:615-618).
void MatmulOp::markWeight(Tensor *A, Tensor *B) {
    if (A->getType() == Tensor::Input && B->getType() == Tensor::Input)
        B->setType(Tensor::Weight);
}

void MatmulOp::dimExtend(Tensor *t) {
    Dim d = t->getDims();
    if (d.size() == 2) {
        d.insert(d.begin(), 1);
        t->setDims(d);
    }
}

bool MatmulOp::checkValid(const TensorVec &ins) {
    auto A = ins[0], B = ins[1];
    if (A->getType() == Tensor::Weight && B->getType() == Tensor::Weight)
        return false;
    const Dim &a = A->getDims(), &b = B->getDims();
    if (a.size() != 3 || b.size() != 3 || a[0] != b[0])
        return false;
    return (transA ? a[1] : a[2]) == (transB ? b[2] : b[1]);
}

MatmulArgs MatmulOp::getArgs() const {
    const Dim &a = inputs[0]->getDims(), &b = inputs[1]->getDims();
    return MatmulArgs{transA, transB, a[0], transA ? a[2] : a[1], transB ? b[1] : b[2],
                      transA ? a[1] : a[2]};
}

Dim MatmulOp::computeShape() {
    bool ta, tb;
    int b, m, n, k;
    std::tie(ta, tb, b, m, n, k) = getArgs();
    Dim ret = {b, m, n};
    outputs[0]->setDims(ret);
    outputs[0]->setType(Tensor::Input);
    return ret;
}

bool MatmulOp::biasPerBatch() const {
    bool ta, tb;
    int b, m, n, k;
    std::tie(ta, tb, b, m, n, k) = getArgs();
    return bias != nullptr && b > 1 && bias->size() == (size_t)b * n;
}

unsigned MatmulOp::operandFlags() const {
    return (sharedLhs ? PET_HIP_CALL_A_SHARED : 0u) | (biasPerBatch() ? PET_HIP_CALL_BIAS_PER_BATCH : 0u);
}

int MatmulOp::launch(pet_hip_stream_t stream) {
    bool ta, tb;
    int b, m, n, k;
    std::tie(ta, tb, b, m, n, k) = getArgs();
    if (algo != 0 || operandFlags() != 0)
        return launchFused(stream, nullptr, act, outputs[0]->devicePtr(), 0);
    return pet_hip_bmm_f32(ta, tb, b, m, n, k, inputs[0]->devicePtr(), inputs[1]->devicePtr(),
                           outputs[0]->devicePtr(), bias ? bias->devicePtr() : nullptr, (int)act,
                           stream);
}

int MatmulOp::launchFused(pet_hip_stream_t stream, const float *residual, ActType finalAct,
                          float *out, unsigned flags) {
    if (residual != nullptr && act != None)
        return PET_HIP_ERR_INVALID;
    bool ta, tb;
    int b, m, n, k;
    std::tie(ta, tb, b, m, n, k) = getArgs();
    const float *A = sharedLhs ? sharedLhs->devicePtr() : inputs[0]->devicePtr();
    return pet_hip_bmm_ex_f32(ta, tb, b, m, n, k, A, inputs[1]->devicePtr(), out,
                              bias ? bias->devicePtr() : nullptr, residual, (int)finalAct,
                              flags | operandFlags() | PET_HIP_CONV_ALGO(algo), stream);
}

bool MatmulOp::accumulates() const {
    if (operandFlags() != 0)
        return false; // these forms never add partial sums into an initialised output
    bool ta, tb;
    int b, m, n, k, yes = 0;
    std::tie(ta, tb, b, m, n, k) = getArgs();
    return pet_hip_bmm_accumulates(ta, tb, b, m, n, k, &yes) == PET_HIP_OK && yes != 0;
}

double MatmulOp::perf(PerfEngine *pe, int rounds, int warmupRounds) {
    MatmulArgs args = getArgs();
    if (pe->checkOpPerf(Matmul, args)) {
        algo = pe->getMatmulAlgo(args);
        return pe->getOpPerf(Matmul, args);
    }
    bool ta, tb;
    int b, m, n, k;
    std::tie(ta, tb, b, m, n, k) = args;
    float *A = pe->getMatA((size_t)b * m * k), *B = pe->getMatB((size_t)b * k * n);
    float *C = pe->getMatC((size_t)b * m * n);
    MatmulResult best{INFINITY, true, 0};
    if (A && B && C) {
        // the search of ConvOp::perf (the reference loops over cuBLAS algorithms here,
        // src/Graph/operator.cc:756-815)
        auto run = [&](int a, int rds, int warm) {
            return timeFn(
                [&](pet_hip_stream_t st) {
                    return pet_hip_bmm_ex_f32(ta, tb, b, m, n, k, A, B, C, nullptr, nullptr,
                                              (int)act, PET_HIP_CONV_ALGO(a), st);
                },
                rds, warm);
        };
        best.time = run(0, rounds, warmupRounds);
        static const bool tune = getenv("PET_HOST_NO_ALGO_SEARCH") == nullptr;
        const int quick = std::max(10, rounds / 4);
        for (int a = 1; tune && !ta && !tb && k % 32 == 0 && a < PET_HIP_CONV_ALGO_COUNT; ++a) {
            double t = run(a, quick, std::min(warmupRounds, 10));
            if (!(t < 0.97 * best.time))
                continue;
            t = run(a, rounds, std::min(warmupRounds, 20));
            if (t < 0.97 * best.time) {
                best.time = t;
                best.algo = a;
            }
        }
    }
    pe->saveOpPerf(Matmul, args, best);
    algo = best.algo;
    return best.time;
}

std::string MatmulOp::toString() const {
    std::ostringstream os;
    os << "Matmul([" << (transA ? "A^T" : "A") << "," << (transB ? "B^T" : "B")
       << ",act=" << (int)act << "]";
    if (inputs.size() == 2) {
        bool ta, tb;
        int b, m, n, k;
        std::tie(ta, tb, b, m, n, k) = getArgs();
        os << "," << tensorTag("A", inputs[0]) << "," << tensorTag("B", inputs[1]) << ","
           << tensorTag("C", outputs[0]) << ", bmnk: " << b << ", " << m << ", " << n << ", " << k;
    }
    os << ")";
    return os.str();
}

// ---- Pad / Slice ------------------------------------------------------------------

PadOp::PadOp(Tensor *input, Tensor *output, const Dim &begin, const Dim &end)
    : Operator(Pad, {input}, {output}), begin(begin), end(end) {
    PET_OPERANDS_VALID(checkValid({input}));
    computeShape();
    initHash();
}
PadOp::PadOp(Tensor *input, const Dim &begin, const Dim &end)
    : PadOp(input, new Tensor(), begin, end) {}
PadOp::PadOp(const Dim &begin, const Dim &end) : Operator(Pad), begin(begin), end(end) {
    initHash();
}

void PadOp::initHash() { hash = hashPack(hashDims(hashDims(type, begin), end)); }

bool PadOp::checkValid(const TensorVec &ins) {
    const Dim &d = ins[0]->getDims();
    if (begin.size() != d.size() || end.size() != d.size())
        return false;
    for (size_t i = 0; i < d.size(); ++i)
        if (begin[i] < 0 || end[i] < 0)
            return false;
    return true;
}

Dim PadOp::computeShape() {
    Dim d = inputs[0]->getDims();
    for (size_t i = 0; i < d.size(); ++i)
        d[i] += begin[i] + end[i];
    outputs[0]->setDims(d);
    outputs[0]->setType(inputs[0]->getType());
    return d;
}

int PadOp::launch(pet_hip_stream_t stream) {
    const Dim &d = inputs[0]->getDims();
    return pet_hip_pad(inputs[0]->devicePtr(), outputs[0]->devicePtr(), d.data(), begin.data(),
                       end.data(), (int)d.size(), stream);
}

double PadOp::perf(PerfEngine *, int rounds, int warmupRounds) {
    return timeLaunches(std::min(rounds, 50), std::min(warmupRounds, 10));
}

std::string PadOp::toString() const {
    std::ostringstream os;
    os << "Pad(begin=" << dimToString(begin) << ",end=" << dimToString(end) << ")";
    return os.str();
}

SliceOp::SliceOp(Tensor *input, Tensor *output, const Dim &begin, const Dim &end)
    : Operator(Slice, {input}, {output}), begin(begin), end(end) {
    PET_OPERANDS_VALID(checkValid({input}));
    computeShape();
    initHash();
}
SliceOp::SliceOp(Tensor *input, const Dim &begin, const Dim &end)
    : SliceOp(input, new Tensor(), begin, end) {}
SliceOp::SliceOp(const Dim &begin, const Dim &end) : Operator(Slice), begin(begin), end(end) {
    initHash();
}

void SliceOp::initHash() { hash = hashPack(hashDims(hashDims(type, begin), end)); }

bool SliceOp::checkValid(const TensorVec &ins) {
    const Dim &d = ins[0]->getDims();
    if (begin.size() != d.size() || end.size() != d.size())
        return false;
    for (size_t i = 0; i < d.size(); ++i)
        if (begin[i] < 0 || end[i] < 0 || d[i] < begin[i] + end[i])
            return false;
    return true;
}

Dim SliceOp::computeShape() {
    Dim d = inputs[0]->getDims();
    for (size_t i = 0; i < d.size(); ++i)
        d[i] -= begin[i] + end[i];
    outputs[0]->setDims(d);
    outputs[0]->setType(inputs[0]->getType());
    return d;
}

int SliceOp::launch(pet_hip_stream_t stream) {
    const Dim &d = inputs[0]->getDims();
    return pet_hip_slice(inputs[0]->devicePtr(), outputs[0]->devicePtr(), d.data(), begin.data(),
                         end.data(), (int)d.size(), stream);
}

double SliceOp::perf(PerfEngine *, int rounds, int warmupRounds) {
    return timeLaunches(std::min(rounds, 50), std::min(warmupRounds, 10));
}

std::string SliceOp::toString() const {
    std::ostringstream os;
    os << "Slice(begin=" << dimToString(begin) << ",end=" << dimToString(end) << ")";
    return os.str();
}

// ---- Concat / Split ---------------------------------------------------------------

ConcatOp::ConcatOp(TensorVec ins, Tensor *output, int dim)
    : Operator(Concat, std::move(ins), {output}), dim(dim) {
    computeShape();
    initHash();
}
ConcatOp::ConcatOp(TensorVec ins, int dim) : ConcatOp(std::move(ins), new Tensor(), dim) {}
ConcatOp::ConcatOp(int dim) : Operator(Concat), dim(dim) { initHash(); }

void ConcatOp::initHash() { hash = hashPack(hashAppend(type, dim)); }

bool ConcatOp::checkValid(const TensorVec &ts) {
    if (ts.empty())
        return false;
    const Dim &first = ts[0]->getDims();
    if (dim < 0 || dim >= (int)first.size())
        return false;
    for (auto t : ts) {
        if (t->getType() != ts[0]->getType() || t->getDims().size() != first.size())
            return false;
        for (size_t i = 0; i < first.size(); ++i)
            if ((int)i != dim && t->getDims()[i] != first[i])
                return false;
    }
    return true;
}

Dim ConcatOp::computeShape() {
    Dim ret = inputs[0]->getDims();
    ret[dim] = 0;
    for (auto t : inputs)
        ret[dim] += t->getDims()[dim];
    outputs[0]->setDims(ret);
    outputs[0]->setType(inputs[0]->getType());
    return ret;
}

int ConcatOp::launch(pet_hip_stream_t stream) {
    std::vector<const float *> ptrs;
    std::vector<int> sizes;
    for (auto t : inputs) {
        ptrs.push_back(t->devicePtr());
        sizes.push_back(t->getDims()[dim]);
    }
    const Dim &od = outputs[0]->getDims();
    return pet_hip_concat(ptrs.data(), (int)ptrs.size(), outputs[0]->devicePtr(), od.data(),
                          (int)od.size(), dim, sizes.data(), stream);
}

// On dim 0 the graph runtime makes the parts views of the whole (no kernel).
double ConcatOp::perf(PerfEngine *, int rounds, int warmupRounds) {
    if (dim == 0)
        return 0.0;
    return timeLaunches(std::min(rounds, 50), std::min(warmupRounds, 10));
}

std::string ConcatOp::toString() const {
    std::ostringstream os;
    os << "Concat(dim=" << dim << ",n=" << inputs.size() << ")";
    return os.str();
}

SplitOp::SplitOp(Tensor *input, const TensorVec &outs, int dim, const std::vector<int> &sizes)
    : Operator(Split, {input}, outs), dim(dim), num(-1), sizes(sizes) {
    computeShapeV();
    initHash();
}
SplitOp::SplitOp(Tensor *input, int dim, int num)
    : Operator(Split, {input}, {}), dim(dim), num(num) {
    for (int i = 0; i < num; ++i)
        outputs.push_back(new Tensor());
    computeShapeV();
    initHash();
}
SplitOp::SplitOp(Tensor *input, int dim, const std::vector<int> &sizes)
    : Operator(Split, {input}, {}), dim(dim), num(-1), sizes(sizes) {
    for (size_t i = 0; i < sizes.size(); ++i)
        outputs.push_back(new Tensor());
    computeShapeV();
    initHash();
}
SplitOp::SplitOp(int dim, int num) : Operator(Split), dim(dim), num(num) { initHash(); }
SplitOp::SplitOp(int dim, const std::vector<int> &sizes)
    : Operator(Split), dim(dim), num(-1), sizes(sizes) {
    initHash();
}

void SplitOp::initHash() {
    hash = hashAppend(hashAppend(type, dim), num);
    hash = hashPack(hashDims(hash, sizes));
}

// `sizes` are proportions: part i gets dim / sum(sizes) * sizes[i]
// (src/Graph/operator.cc:2085-2094); an equal split when only `num` is known.
std::vector<Dim> SplitOp::computeShapeV() {
    auto fail = [&]() {
        for (auto t : outputs)
            t->setInvalid();
        return std::vector<Dim>();
    };
    if (sizes.empty()) {
        if (num <= 0)
            return fail();
        sizes.assign(num, 1);
    }
    const Dim &in = inputs[0]->getDims();
    int total = std::accumulate(sizes.begin(), sizes.end(), 0);
    if (dim < 0 || dim >= (int)in.size() || total <= 0 || in[dim] % total != 0 ||
        outputs.size() != sizes.size())
        return fail();
    std::vector<Dim> ret;
    for (size_t i = 0; i < outputs.size(); ++i) {
        Dim d = in;
        d[dim] = in[dim] / total * sizes[i];
        ret.push_back(d);
        outputs[i]->setDims(d);
        if (outputs[i]->getType() != Tensor::NotCounted)
            outputs[i]->setType(inputs[0]->getType());
    }
    return ret;
}

Dim SplitOp::computeShape() {
    auto v = computeShapeV();
    return v.empty() ? Dim{} : v[0];
}

bool SplitOp::computeShape(const TensorVec &ins, const TensorVec &outs) {
    if (ins.size() != 1 || ins[0] == nullptr || (num == -1 && outs.empty()))
        return false;
    if (ins[0]->getDims().size() <= (size_t)dim)
        return false;
    inputs = ins;
    outputs = outs;
    return !computeShapeV().empty();
}

Tensor *SplitOp::compute() {
    auto v = computeV();
    return v.empty() ? nullptr : v[0];
}

TensorVec SplitOp::computeV() {
    if (Operator::compute() == nullptr)
        return {};
    return outputs;
}

std::pair<std::vector<DimRange>, std::function<bool()>> SplitOp::compute(size_t idx,
                                                                         DimRange dr) {
    if (dr.notValid() || idx >= outputs.size())
        return {};
    if (dr.isEmpty())
        return {{DimRange::getEmpty()}, []() { return true; }};
    auto whole = [this]() { return !computeV().empty(); };
    if (!dr.isSinglePos())
        return {{DimRange::getAllPos()}, whole};
    Dim src = dr.getBegin();
    if (src.size() != inputs[0]->getDims().size())
        return {};
    for (size_t i = 0; i < idx; ++i)
        src[dim] += outputs[i]->getDims()[dim];
    return {{DimRange(src)}, whole};
}

int SplitOp::launch(pet_hip_stream_t stream) {
    std::vector<float *> ptrs;
    std::vector<int> outSizes;
    for (auto t : outputs) {
        if (!t->isValid())
            return PET_HIP_ERR_INVALID;
        ptrs.push_back(t->devicePtr());
        outSizes.push_back(t->getDims()[dim]);
    }
    const Dim &in = inputs[0]->getDims();
    return pet_hip_split(inputs[0]->devicePtr(), ptrs.data(), (int)ptrs.size(), in.data(),
                         (int)in.size(), dim, outSizes.data(), stream);
}

double SplitOp::perf(PerfEngine *, int rounds, int warmupRounds) {
    if (dim == 0)
        return 0.0;
    return timeLaunches(std::min(rounds, 50), std::min(warmupRounds, 10));
}

std::string SplitOp::toString() const {
    std::ostringstream os;
    os << "Split(dim=" << dim << ",sizes=" << dimToString(sizes.empty() ? Dim{num} : sizes) << ")";
    return os.str();
}

// ---- Transpose ----------------------------------------------------------------------

std::string PermItem::toString() const {
    if (isSingle())
        return std::to_string(items[0]);
    std::string s = "{";
    for (size_t i = 0; i < items.size(); ++i)
        s += (i ? "," : "") + std::to_string(items[i]);
    return s + "}";
}

std::vector<int> Perm::asVector() const {
    std::vector<int> v;
    for (auto &pi : perm)
        v.insert(v.end(), pi.items.begin(), pi.items.end());
    return v;
}

std::string Perm::toString() const {
    std::string s = "{";
    for (size_t i = 0; i < perm.size(); ++i)
        s += (i ? "," : "") + perm[i].toString();
    return s + "}";
}

TransposeOp::TransposeOp(Tensor *input, Tensor *output, const Perm &before, const Perm &after,
                         int factor, TransType trans_type)
    : Operator(Transpose, {input}, {output}), before(before), after(after), split(-1),
      factor(factor), trans_type(trans_type) {
    for (size_t i = 0; i < before.size(); ++i)
        if (!before[i].isSingle()) {
            split = (int)i;
            break;
        }
    PET_OPERANDS_VALID(checkValid({input}));
    initHash();
    computeShape();
}

TransposeOp::TransposeOp(Tensor *input, Tensor *output, int split, const Perm &after, int factor,
                         TransType trans_type)
    : Operator(Transpose, {input}, {output}), before({}), after(after), split(split),
      factor(factor), trans_type(trans_type) {
    initHash();
    setParam((int)input->getDims().size());
    PET_OPERANDS_VALID(checkValid({input}));
    computeShape();
}

TransposeOp::TransposeOp(Tensor *input, int split, const Perm &after, int factor,
                         TransType trans_type)
    : TransposeOp(input, new Tensor(), split, after, factor, trans_type) {}

TransposeOp::TransposeOp(int split, const Perm &after, int factor, TransType trans_type)
    : Operator(Transpose), before({}), after(after), split(split), factor(factor),
      trans_type(trans_type) {
    initHash();
    int rank = 0;
    for (int v : after.asVector())
        rank = std::max(rank, v + 1);
    setParam(rank);
}

TransposeOp::TransposeOp(const TransposeOp &rhs)
    : Operator(rhs), before(rhs.before), after(rhs.after), split(rhs.split), factor(rhs.factor),
      trans_type(rhs.trans_type), trans_pos(rhs.trans_pos), padding_h(rhs.padding_h),
      padding_w(rhs.padding_w) {}

// Builds `before` as the identity with the split dim doubled, and renumbers
// `after`: entries past the split move up by one, -1 becomes the new dim
// (include/operator.h:1124-1144 of the reference).
void TransposeOp::setParam(int dimSz) {
    int idx = 0;
    for (int i = 0; i < dimSz; ++i) {
        if (i == split) {
            before.getPerm().emplace_back(PermItem({idx, idx + 1}));
            idx += 2;
        } else {
            before.getPerm().emplace_back(idx++);
        }
    }
    if (split < 0)
        return;
    for (size_t i = 0; i < after.size(); ++i)
        for (int &item : after[i].getVec()) {
            if (item > split)
                item += 1;
            else if (item == -1)
                item = split + 1;
        }
}

void TransposeOp::initHash() {
    hash = hashAppend(hashAppend(type, (uint64_t)(int64_t)factor), (uint64_t)(int64_t)split);
    int merge = -1;
    for (size_t i = 0; i < after.size(); ++i)
        if (!after[i].isSingle())
            merge = (int)i;
    hash = hashAppend(hash, (uint64_t)(int64_t)merge);
    for (int x : after.asVector())
        hash = hashAppend(hash, (uint64_t)(int64_t)x);
}

bool TransposeOp::checkValid(const TensorVec &ins) {
    if (split != -1 && factor == 0)
        return false;
    auto b = before.asVector(), a = after.asVector();
    if (b.size() != a.size() || before.size() != ins[0]->getDims().size())
        return false;
    std::sort(a.begin(), a.end());
    for (size_t i = 0; i < b.size(); ++i)
        if (b[i] != (int)i || a[i] != (int)i)
            return false;
    auto multi = [](const Perm &p) {
        int c = 0;
        for (size_t i = 0; i < p.size(); ++i)
            c += !p[i].isSingle();
        return c;
    };
    return multi(before) <= 1 && multi(after) <= 1;
}

// The split dim d becomes (d / f, f) for f > 0 and (-f, d / -f) for f < 0.
bool TransposeOp::flatDims(Dim &flat) const {
    const Dim &in = inputs[0]->getDims();
    flat.clear();
    for (size_t i = 0; i < before.size(); ++i) {
        if (before[i].isSingle()) {
            flat.push_back(in[i]);
            continue;
        }
        int f = factor > 0 ? factor : -factor;
        if (f == 0 || in[i] % f != 0 || in[i] < f)
            return false;
        if (factor > 0) {
            flat.push_back(in[i] / f);
            flat.push_back(f);
        } else {
            flat.push_back(f);
            flat.push_back(in[i] / f);
        }
    }
    return true;
}

bool TransposeOp::corrected() const {
    if (trans_pos == NonePos)
        return false;
    switch (trans_type) {
    case N2H:
    case H2N:
        return padding_h > 0;
    case N2W:
    case W2N:
        return padding_w > 0;
    default:
        return false;
    }
}

// Micro-op list. Pairing of the correction parameters: a spatial split that
// goes in front of the convolution (H2N / W2N, Pre) gives each half `padding`
// halo rows (copys) and the merge after it (N2H / N2W, Post) drops them (dels);
// a merge in front (N2H / N2W, Pre) separates the images by `padding` zero rows
// (pad) and the split after it (H2N / W2N, Post) skips them (extr).
std::vector<std::shared_ptr<TransBasic>> TransposeOp::getTTParam() const {
    int extr = 0, pad = 0, copys = 0, dels = 0;
    if (corrected()) {
        int p = (trans_type == N2H || trans_type == H2N) ? padding_h : padding_w;
        bool splitsSpatial = trans_type == H2N || trans_type == W2N;
        if (splitsSpatial)
            (trans_pos == Pre ? copys : extr) = p;
        else
            (trans_pos == Pre ? pad : dels) = p;
    }
    std::vector<std::shared_ptr<TransBasic>> ret;
    const Dim &in = inputs[0]->getDims();
    if (split >= 0) {
        int f = factor > 0 ? factor : -factor;
        int inner;
        if (extr > 0) {
            // the input carries `extr` zero rows between its f (or d/f) blocks
            int blocks = factor > 0 ? 0 : f;
            inner = blocks ? (in[split] + extr) / blocks - extr : f;
        } else {
            inner = factor > 0 ? f : in[split] / f;
        }
        ret.emplace_back(new TransSplit(split, inner, extr, copys));
    }
    ret.emplace_back(new TransReorder(after.asVector()));
    for (size_t i = 0; i < after.size(); ++i)
        if (!after[i].isSingle()) {
            for (size_t j = 0; j + 1 < after[i].getVec().size(); ++j)
                ret.emplace_back(new TransFuse((int)i, pad, dels));
            break;
        }
    return ret;
}

Dim TransposeOp::computeShape() {
    if (corrected()) {
        TransProgram prog;
        if (!TransposeEngine::getInstance().lower(getTTParam(), inputs[0]->getDims(), prog)) {
            outputs[0]->setInvalid();
            return {};
        }
        outputs[0]->setDims(prog.outDims);
        outputs[0]->setType(inputs[0]->getType());
        return prog.outDims;
    }
    Dim flat;
    if (!flatDims(flat)) {
        outputs[0]->setInvalid();
        return {};
    }
    Dim ret(after.size(), 1);
    for (size_t i = 0; i < after.size(); ++i)
        for (int j : after[i].getVec())
            ret[i] *= flat[j];
    outputs[0]->setDims(ret);
    outputs[0]->setType(inputs[0]->getType());
    return ret;
}

int TransposeOp::launch(pet_hip_stream_t stream) {
    if (corrected()) {
        TransProgram prog;
        if (!TransposeEngine::getInstance().lower(getTTParam(), inputs[0]->getDims(), prog))
            return PET_HIP_ERR_INVALID;
        int outDims[PET_HIP_MAX_RANK], outRank = 0;
        return pet_hip_trans_chain(inputs[0]->devicePtr(), outputs[0]->devicePtr(),
                                   prog.inDims.data(), (int)prog.inDims.size(), prog.ops.data(),
                                   prog.nops, prog.perms.data(), outDims, &outRank, stream);
    }
    Dim flat;
    if (!flatDims(flat))
        return PET_HIP_ERR_INVALID;
    auto perm = after.asVector();
    return pet_hip_transpose(inputs[0]->devicePtr(), outputs[0]->devicePtr(), flat.data(),
                             perm.data(), (int)flat.size(), stream);
}

// Weight-side transposes run once outside the timed loop and a transpose that
// follows another one is folded into it, so both cost nothing (the reference's
// rule, src/Graph/operator.cc:2384-2388); everything else is timed.
double TransposeOp::perf(PerfEngine *, int rounds, int warmupRounds) {
    if (inputs[0]->getType() == Tensor::Weight)
        return 0.0;
    Operator *prev = inputs[0]->getOutputOf();
    if (prev != nullptr && prev->getType() == Transpose)
        return 0.0;
    return timeLaunches(std::min(rounds, 50), std::min(warmupRounds, 10));
}

std::string TransposeOp::toString() const {
    std::ostringstream os;
    os << "Transpose[" << hash << "](before=" << before.toString() << ",after=" << after.toString()
       << ",split=" << split << ",factor=" << factor << ",type=" << trans_type
       << ",pos=" << trans_pos << ",pad=[" << padding_h << "," << padding_w << "])";
    return os.str();
}

// ---- Extend -----------------------------------------------------------------------

ExtendOp::ExtendOp(Tensor *input, Tensor *output, int dim, int num)
    : Operator(Extend, {input}, {output}), dim(dim), num(num) {
    computeShape();
    initHash();
}
ExtendOp::ExtendOp(Tensor *input, int dim, int num) : ExtendOp(input, new Tensor(), dim, num) {}
ExtendOp::ExtendOp(int dim, int num) : Operator(Extend), dim(dim), num(num) { initHash(); }

void ExtendOp::initHash() { hash = hashPack(hashAppend(hashAppend(type, dim), num)); }

Dim ExtendOp::computeShape() {
    Dim ret = inputs[0]->getDims();
    ret[dim] *= (num + 1);
    outputs[0]->setDims(ret);
    outputs[0]->setType(inputs[0]->getType());
    return ret;
}

int ExtendOp::launch(pet_hip_stream_t stream) {
    const Dim &d = inputs[0]->getDims();
    return pet_hip_extend(inputs[0]->devicePtr(), outputs[0]->devicePtr(), d.data(),
                          (int)d.size(), dim, num, stream);
}

double ExtendOp::perf(PerfEngine *, int rounds, int warmupRounds) {
    return timeLaunches(std::min(rounds, 50), std::min(warmupRounds, 10));
}

std::string ExtendOp::toString() const {
    std::ostringstream os;
    os << "Extend(dim=" << dim << ",num=" << num << ")";
    return os.str();
}

// ---- element-wise -------------------------------------------------------------------

EltwiseOp::EltwiseOp(OpType type, TensorVec ins, Tensor *output)
    : Operator(type, std::move(ins), {output ? output : new Tensor()}) {
    PET_OPERANDS_VALID(checkValid(inputs));
    if (outputs[0]->getDims().empty())
        computeShape();
    initHash();
}

void EltwiseOp::initHash() { hash = hashPack(type); }

bool EltwiseOp::checkValid(const TensorVec &ins) {
    if (ins.empty() || ins.size() > 8 || ((type == Sub || type == Div) && ins.size() != 2))
        return false;
    for (auto t : ins)
        if (t == nullptr || t->size() == 0)
            return false;
    return true;
}

bool EltwiseOp::computeShape(const TensorVec &ins, const TensorVec &outs) {
    if (outs.size() != 1 || outs[0] == nullptr || !checkValid(ins))
        return false;
    inputs = ins;
    outputs = outs;
    computeShape();
    return true;
}

// Output takes the shape of the largest operand; smaller ones broadcast by
// flat index modulo their size.
Dim EltwiseOp::computeShape() {
    Tensor *big = inputs[0];
    for (auto t : inputs)
        if (t->size() > big->size())
            big = t;
    outputs[0]->setDims(big->getDims());
    outputs[0]->setType(inputs[0]->getType() == Tensor::Weight ? Tensor::Input
                                                                : inputs[0]->getType());
    return big->getDims();
}

int EltwiseOp::launch(pet_hip_stream_t stream) {
    std::vector<const float *> ptrs;
    std::vector<size_t> sizes;
    for (auto t : inputs) {
        ptrs.push_back(t->devicePtr());
        sizes.push_back(t->size());
    }
    int op = type == Add   ? PET_HIP_ADD
             : type == Sub ? PET_HIP_SUB
             : type == Div ? PET_HIP_DIV
                           : PET_HIP_MUL;
    return pet_hip_eltwise(op, ptrs.data(), sizes.data(), (int)ptrs.size(),
                           outputs[0]->devicePtr(), outputs[0]->size(), stream);
}

double EltwiseOp::perf(PerfEngine *, int rounds, int warmupRounds) {
    return timeLaunches(std::min(rounds, 50), std::min(warmupRounds, 10));
}

std::string EltwiseOp::toString() const {
    return getOpName(type) + "(n=" + std::to_string(inputs.size()) + ")";
}

// ---- Pow / BatchNorm ------------------------------------------------------------------

PowOp::PowOp(Tensor *input, Tensor *output, int pow) : Operator(Pow, {input}, {output}), pow(pow) {
    PET_OPERANDS_VALID(checkValid(inputs));
    computeShape();
    initHash();
}
PowOp::PowOp(Tensor *input, int pow) : PowOp(input, new Tensor(), pow) {}
PowOp::PowOp(int pow) : Operator(Pow), pow(pow) { initHash(); }

void PowOp::initHash() { hash = hashPack(hashAppend(type, pow)); }

Dim PowOp::computeShape() {
    outputs[0]->setDims(inputs[0]->getDims());
    outputs[0]->setType(inputs[0]->getType());
    return inputs[0]->getDims();
}

int PowOp::launch(pet_hip_stream_t stream) {
    return pet_hip_pow(inputs[0]->devicePtr(), outputs[0]->devicePtr(), inputs[0]->size(), pow,
                       stream);
}

double PowOp::perf(PerfEngine *, int rounds, int warmupRounds) {
    return timeLaunches(std::min(rounds, 50), std::min(warmupRounds, 10));
}

std::string PowOp::toString() const { return "Pow(pow=" + std::to_string(pow) + ")"; }

BatchNormOp::BatchNormOp(Tensor *input, Tensor *scale, Tensor *bias, Tensor *mean, Tensor *var,
                         Tensor *output, float epsilon, float momentum)
    : Operator(BatchNorm, {input}, {output}), epsilon(epsilon), momentum(momentum), scale(scale),
      bias(bias), mean(mean), var(var) {
    PET_OPERANDS_VALID(checkValid(inputs));
    computeShape();
    initHash();
}
BatchNormOp::BatchNormOp(Tensor *input, Tensor *scale, Tensor *bias, Tensor *mean, Tensor *var,
                         float epsilon, float momentum)
    : BatchNormOp(input, scale, bias, mean, var, new Tensor(), epsilon, momentum) {}
BatchNormOp::BatchNormOp(Tensor *scale, Tensor *bias, Tensor *mean, Tensor *var, float epsilon,
                         float momentum)
    : Operator(BatchNorm), epsilon(epsilon), momentum(momentum), scale(scale), bias(bias),
      mean(mean), var(var) {
    initHash();
}

void BatchNormOp::initHash() { hash = hashPack(type); }

// every per-channel vector has as many elements as the input has channels
bool BatchNormOp::checkValid(const TensorVec &ins) {
    if (ins.size() != 1 || ins[0] == nullptr || ins[0]->getDims().size() < 2)
        return false;
    size_t c = (size_t)ins[0]->getDims()[1];
    for (Tensor *t : {scale, bias, mean, var})
        if (t == nullptr || t->size() != c)
            return false;
    return true;
}

Dim BatchNormOp::computeShape() {
    outputs[0]->setDims(inputs[0]->getDims());
    outputs[0]->setType(Tensor::Input);
    return inputs[0]->getDims();
}

int BatchNormOp::launch(pet_hip_stream_t stream) {
    const Dim &d = inputs[0]->getDims();
    size_t inner = 1;
    for (size_t i = 2; i < d.size(); ++i)
        inner *= (size_t)d[i];
    return pet_hip_batchnorm(inputs[0]->devicePtr(), scale->devicePtr(), bias->devicePtr(),
                             mean->devicePtr(), var->devicePtr(), outputs[0]->devicePtr(),
                             (size_t)d[0], (size_t)d[1], inner, epsilon, stream);
}

double BatchNormOp::perf(PerfEngine *, int rounds, int warmupRounds) {
    return timeLaunches(std::min(rounds, 50), std::min(warmupRounds, 10));
}

std::string BatchNormOp::toString() const {
    std::ostringstream os;
    os << "BatchNorm(in=" << inputs[0]->getHash() << ",out=" << outputs[0]->getHash() << ")";
    return os.str();
}

// ---- Gather / ReduceMean --------------------------------------------------------------

GatherOp::GatherOp(Tensor *data, Tensor *indices, Tensor *output, int axis)
    : Operator(Gather, {data, indices}, {output}), axis(axis) {
    PET_OPERANDS_VALID(checkValid(inputs));
    computeShape();
    initHash();
}
GatherOp::GatherOp(Tensor *data, Tensor *indices, int axis)
    : GatherOp(data, indices, new Tensor(), axis) {}

void GatherOp::initHash() { hash = hashPack(hashAppend(type, axis)); }

bool GatherOp::checkValid(const TensorVec &ins) {
    return ins.size() == 2 && ins[0] && ins[1] && axis >= 0 &&
           axis < (int)ins[0]->getDims().size();
}

Dim GatherOp::computeShape() {
    Dim dim = inputs[1]->getDims();
    const Dim &data = inputs[0]->getDims();
    for (size_t i = 0; i < data.size(); ++i)
        if ((int)i != axis)
            dim.push_back(data[i]);
    outputs[0]->setDims(dim);
    outputs[0]->setType(Tensor::Input);
    return dim;
}

int GatherOp::launch(pet_hip_stream_t stream) {
    const Dim &d = inputs[0]->getDims();
    size_t pre = 1, post = 1;
    for (int i = 0; i < axis; ++i)
        pre *= (size_t)d[i];
    for (size_t i = axis + 1; i < d.size(); ++i)
        post *= (size_t)d[i];
    return pet_hip_gather(inputs[0]->devicePtr(), inputs[1]->devicePtr(), 1,
                          outputs[0]->devicePtr(), pre, (size_t)d[axis], post, inputs[1]->size(),
                          stream);
}

double GatherOp::perf(PerfEngine *, int rounds, int warmupRounds) {
    return timeLaunches(std::min(rounds, 50), std::min(warmupRounds, 10));
}

std::string GatherOp::toString() const {
    std::ostringstream os;
    os << "Gather(data=" << inputs[0]->getHash() << ",indices=" << inputs[1]->getHash()
       << ",out=" << outputs[0]->getHash() << ",axis=" << axis << ")";
    return os.str();
}

ReduceMeanOp::ReduceMeanOp(Tensor *input, Tensor *output, int axis)
    : Operator(ReduceMean, {input}, {output}), axis(axis) {
    PET_OPERANDS_VALID(checkValid(inputs));
    computeShape();
    initHash();
}
ReduceMeanOp::ReduceMeanOp(Tensor *input, int axis) : ReduceMeanOp(input, new Tensor(), axis) {}

void ReduceMeanOp::initHash() { hash = hashPack(hashAppend(type, axis)); }

bool ReduceMeanOp::checkValid(const TensorVec &ins) {
    return ins.size() == 1 && ins[0] && axis >= 0 && axis < (int)ins[0]->getDims().size();
}

Dim ReduceMeanOp::computeShape() {
    Dim dim = inputs[0]->getDims();
    dim[axis] = 1;
    outputs[0]->setDims(dim);
    outputs[0]->setType(inputs[0]->getType());
    return dim;
}

int ReduceMeanOp::launch(pet_hip_stream_t stream) {
    const Dim &d = inputs[0]->getDims();
    size_t outer = 1, inner = 1;
    for (int i = 0; i < axis; ++i)
        outer *= (size_t)d[i];
    for (size_t i = axis + 1; i < d.size(); ++i)
        inner *= (size_t)d[i];
    return pet_hip_reduce_mean(inputs[0]->devicePtr(), outputs[0]->devicePtr(), outer,
                               (size_t)d[axis], inner, stream);
}

double ReduceMeanOp::perf(PerfEngine *, int rounds, int warmupRounds) {
    return timeLaunches(std::min(rounds, 50), std::min(warmupRounds, 10));
}

std::string ReduceMeanOp::toString() const {
    return "ReduceMean(axis=" + std::to_string(axis) + ")";
}

// ---- Activation / Pool / Softmax / LayerNorm / Reshape -----------------------------

ActivationOp::ActivationOp(Tensor *input, Tensor *output, ActType act)
    : Operator(Activation, {input}, {output}), actType(act) {
    computeShape();
    initHash();
}
ActivationOp::ActivationOp(Tensor *input, ActType act)
    : ActivationOp(input, new Tensor(), act) {}
ActivationOp::ActivationOp(ActType act) : Operator(Activation), actType(act) { initHash(); }

void ActivationOp::initHash() { hash = hashPack(hashAppend(type, actType)); }

Dim ActivationOp::computeShape() {
    outputs[0]->setDims(inputs[0]->getDims());
    outputs[0]->setType(inputs[0]->getType());
    return inputs[0]->getDims();
}

int ActivationOp::launch(pet_hip_stream_t stream) {
    return pet_hip_activation(inputs[0]->devicePtr(), outputs[0]->devicePtr(), inputs[0]->size(),
                              (int)actType, stream);
}

double ActivationOp::perf(PerfEngine *, int rounds, int warmupRounds) {
    return timeLaunches(std::min(rounds, 50), std::min(warmupRounds, 10));
}

std::string ActivationOp::toString() const {
    return "Activation(act=" + std::to_string((int)actType) + ")";
}

PoolOp::PoolOp(OpType type, Tensor *input, Tensor *output, int kh, int kw, int dh, int dw, int ph,
               int pw, int sh, int sw)
    : Operator(type, {input}, {output}), kh(kh), kw(kw), dh(dh), dw(dw), ph(ph), pw(pw), sh(sh),
      sw(sw) {
    PET_OPERANDS_VALID(checkValid({input}));
    computeShape();
    initHash();
}

PoolOp::PoolOp(const PoolOp &rhs)
    : Operator(rhs), kh(rhs.kh), kw(rhs.kw), dh(rhs.dh), dw(rhs.dw), ph(rhs.ph), pw(rhs.pw),
      sh(rhs.sh), sw(rhs.sw) {}

AvgPoolOp::AvgPoolOp(Tensor *input, Tensor *output)
    : PoolOp(AvgPool, input, output, input->getDims()[2], input->getDims()[3], 1, 1, 0, 0, 1, 1) {}

void PoolOp::initHash() {
    hash = type;
    for (int v : {kh, kw, dh, dw, ph, pw, sh, sw})
        hash = hashAppend(hash, v);
    hash = hashPack(hash);
}

bool PoolOp::checkValid(const TensorVec &ins) { return ins[0]->getDims().size() == 4; }

Dim PoolOp::computeShape() {
    const Dim &in = inputs[0]->getDims();
    int oh = (in[2] + 2 * ph - dh * (kh - 1) - 1) / sh + 1;
    int ow = (in[3] + 2 * pw - dw * (kw - 1) - 1) / sw + 1;
    Dim ret = {in[0], in[1], oh, ow};
    outputs[0]->setDims(ret);
    outputs[0]->setType(inputs[0]->getType());
    return ret;
}

int PoolOp::launch(pet_hip_stream_t stream) {
    const Dim &in = inputs[0]->getDims();
    return pet_hip_pool2d(inputs[0]->devicePtr(), outputs[0]->devicePtr(), in[0], in[1], in[2],
                          in[3], kh, kw, ph, pw, sh, sw, dh, dw, type == MaxPool ? 0 : 1, stream);
}

int PoolOp::launchFused(pet_hip_stream_t stream, const float *residual, ActType finalAct,
                        float *out, unsigned flags) {
    if (residual != nullptr || finalAct != None)
        return PET_HIP_ERR_INVALID;
    const Dim &in = inputs[0]->getDims();
    return pet_hip_pool2d_ex(inputs[0]->devicePtr(), out, in[0], in[1], in[2], in[3], kh, kw, ph,
                             pw, sh, sw, dh, dw, type == MaxPool ? 0 : 1, flags, stream);
}

double PoolOp::perf(PerfEngine *pe, int rounds, int warmupRounds) {
    PoolArgs args = getArgs();
    if (pe && pe->checkOpPerf(type, args))
        return pe->getOpPerf(type, args);
    double ms = timeLaunches(std::min(rounds, 50), std::min(warmupRounds, 10));
    if (pe)
        pe->saveOpPerf(type, args, (float)ms);
    return ms;
}

std::string PoolOp::toString() const {
    std::ostringstream os;
    os << getOpName(type) << "(k=[" << kh << "," << kw << "],p=[" << ph << "," << pw << "],s=["
       << sh << "," << sw << "],d=[" << dh << "," << dw << "])";
    return os.str();
}

SoftmaxOp::SoftmaxOp(Tensor *input, Tensor *output, int axis)
    : Operator(Softmax, {input}, {output}), axis(axis) {
    PET_OPERANDS_VALID(checkValid({input}));
    computeShape();
    initHash();
}

void SoftmaxOp::initHash() { hash = hashPack(hashAppend(type, axis)); }

bool SoftmaxOp::checkValid(const TensorVec &ins) {
    int rank = (int)ins[0]->getDims().size();
    return rank > 0 && (axis == rank - 1 || axis == -1);
}

Dim SoftmaxOp::computeShape() {
    outputs[0]->setDims(inputs[0]->getDims());
    outputs[0]->setType(inputs[0]->getType());
    return inputs[0]->getDims();
}

int SoftmaxOp::launch(pet_hip_stream_t stream) {
    size_t cols = (size_t)inputs[0]->getDims().back();
    return pet_hip_softmax(inputs[0]->devicePtr(), outputs[0]->devicePtr(),
                           inputs[0]->size() / cols, cols, stream);
}

double SoftmaxOp::perf(PerfEngine *, int rounds, int warmupRounds) {
    return timeLaunches(std::min(rounds, 50), std::min(warmupRounds, 10));
}

std::string SoftmaxOp::toString() const { return "Softmax(axis=" + std::to_string(axis) + ")"; }

LayerNormOp::LayerNormOp(Tensor *input, Tensor *output, Tensor *gamma, Tensor *beta, float eps)
    : Operator(LayerNorm, {input}, {output}), gamma(gamma), beta(beta), eps(eps) {
    computeShape();
    initHash();
}

void LayerNormOp::initHash() { hash = hashPack(type); }

Dim LayerNormOp::computeShape() {
    outputs[0]->setDims(inputs[0]->getDims());
    outputs[0]->setType(inputs[0]->getType());
    return inputs[0]->getDims();
}

int LayerNormOp::launch(pet_hip_stream_t stream) {
    size_t cols = (size_t)inputs[0]->getDims().back();
    return pet_hip_layernorm(inputs[0]->devicePtr(), gamma ? gamma->devicePtr() : nullptr,
                             beta ? beta->devicePtr() : nullptr, outputs[0]->devicePtr(),
                             inputs[0]->size() / cols, cols, eps, stream);
}

double LayerNormOp::perf(PerfEngine *, int rounds, int warmupRounds) {
    return timeLaunches(std::min(rounds, 50), std::min(warmupRounds, 10));
}

std::string LayerNormOp::toString() const { return "LayerNorm()"; }

ReshapeOp::ReshapeOp(OpType type, Tensor *input, Tensor *output)
    : Operator(type, {input}, {output}) {
    initHash();
}
ReshapeOp::ReshapeOp(Tensor *input, Tensor *output) : ReshapeOp(Reshape, input, output) {}

void ReshapeOp::initHash() { hash = hashPack(type); }

// Always valid, as in the reference (include/operator.h:1788): callers build the
// operator first and give the output its dims afterwards
// (src/Mutant/generator.cc:1455-1457). launch() rejects a size mismatch.
bool ReshapeOp::checkValid(const TensorVec &) { return true; }

Dim ReshapeOp::computeShape() {
    outputs[0]->setType(inputs[0]->getType());
    return outputs[0]->getDims();
}

Dim IdentityOp::computeShape() {
    outputs[0]->setDims(inputs[0]->getDims());
    outputs[0]->setType(inputs[0]->getType());
    return inputs[0]->getDims();
}

int ReshapeOp::launch(pet_hip_stream_t stream) {
    if (inputs[0]->size() != outputs[0]->size())
        return PET_HIP_ERR_INVALID;
    float *src = inputs[0]->devicePtr(), *dst = outputs[0]->devicePtr();
    if (src == dst)
        return PET_HIP_OK; // the runtime made the output a view of the input
    return pet_hip_memcpy_d2d(dst, src, inputs[0]->size() * sizeof(float), stream);
}

double ReshapeOp::perf(PerfEngine *, int, int) { return 0.0; }

std::string ReshapeOp::toString() const {
    return getOpName(type) + "(" + dimToString(inputs[0]->getDims()) + "->" +
           dimToString(outputs[0]->getDims()) + ")";
}

// ---- band matrix products --------------------------------------------------------
G2BMMOp::G2BMMOp(Tensor *A, Tensor *B, Tensor *C, int width, int dilation, Tensor *bias,
                 ActType act)
    : Operator(G2BMM, {A, B}, {C}), width(width), dilation(dilation), bias(bias), act(act) {
    if (A->getType() == Tensor::Input && B->getType() == Tensor::Input)
        B->setType(Tensor::Weight);
    PET_OPERANDS_VALID(checkValid({A, B}));
    computeShape();
    initHash();
}

G2BMMOp::G2BMMOp(Tensor *A, Tensor *B, int width, int dilation, Tensor *bias, ActType act)
    : G2BMMOp(A, B, new Tensor(), width, dilation, bias, act) {}

G2BMMOp::G2BMMOp(int width, int dilation, Tensor *bias, ActType act)
    : Operator(G2BMM), width(width), dilation(dilation), bias(bias), act(act) {
    initHash();
}

G2BMMGBMMLArgs G2BMMOp::getArgs() const {
    if (inputs.empty())
        return G2BMMGBMMLArgs{0, 0, 0, width, dilation};
    const Dim &a = inputs[0]->getDims();
    return G2BMMGBMMLArgs{a[0], a[1], a[2], width, dilation};
}

void G2BMMOp::initHash() {
    auto [b, m, k, w, d] = getArgs();
    hash = type;
    for (int v : {b, m, k, w, d})
        hash = hashAppend(hash, (uint64_t)(int64_t)v);
    hash = hashPack(hash);
}

bool G2BMMOp::checkValid(const TensorVec &ins) {
    const Tensor *A = ins[0], *B = ins[1];
    if (A->getType() == Tensor::Weight && B->getType() == Tensor::Weight)
        return false;
    return A->getDims().size() == 3 && A->getDims() == B->getDims() && width >= 0;
}

Dim G2BMMOp::computeShape() {
    const Dim &a = inputs[0]->getDims();
    Dim ret = {a[0], a[1], 2 * width + 1};
    outputs[0]->setDims(ret);
    outputs[0]->setType(Tensor::Input);
    return ret;
}

int G2BMMOp::launch(pet_hip_stream_t stream) {
    const Dim &a = inputs[0]->getDims();
    return pet_hip_g2bmm_f32(inputs[0]->devicePtr(), inputs[1]->devicePtr(),
                             outputs[0]->devicePtr(), a[0], a[1], a[2], width, dilation, stream);
}

// Timed on the PerfEngine's scratch operands and memoised per (b, m, k, width, dilation),
// as the reference times _sg2bmm (src/Graph/operator.cc:1424-1468).
double G2BMMOp::perf(PerfEngine *pe, int rounds, int warmupRounds) {
    G2BMMGBMMLArgs args = getArgs();
    if (pe->checkOpPerf(G2BMM, args))
        return pe->getOpPerf(G2BMM, args);
    auto [b, m, k, w, d] = args;
    double ms = INFINITY;
    if (b > 0 && m > 0 && k > 0) {
        float *A = pe->getMatA((size_t)b * m * k), *B = pe->getMatB((size_t)b * m * k);
        float *C = pe->getMatC((size_t)b * m * (2 * w + 1));
        if (A && B && C)
            ms = timeFn(
                [&](pet_hip_stream_t st) { return pet_hip_g2bmm_f32(A, B, C, b, m, k, w, d, st); },
                rounds, warmupRounds);
    }
    pe->saveOpPerf(G2BMM, args, (float)ms);
    return pe->getOpPerf(G2BMM, args);
}

std::string G2BMMOp::toString() const {
    std::ostringstream os;
    os << "G2BMM[" << hash << "](";
    if (inputs.size() == 2)
        os << dimToString(inputs[0]->getDims()) << "," << dimToString(inputs[1]->getDims()) << ",";
    os << "width=" << width << ",dilation=" << dilation << ",act=" << act;
    if (inputs.size() == 2)
        os << "," << tensorTag("A", inputs[0]) << "," << tensorTag("B", inputs[1]) << ","
           << tensorTag("C", outputs[0]);
    os << ")";
    return os.str();
}

GBMMLOp::GBMMLOp(Tensor *A, Tensor *B, Tensor *C, int dilation, Tensor *bias, ActType act)
    : Operator(GBMML, {A, B}, {C}), dilation(dilation), bias(bias), act(act) {
    // both operands stay inputs: in attention neither is a constant
    // (src/Graph/operator.cc:1489-1493)
    PET_OPERANDS_VALID(checkValid({A, B}));
    computeShape();
    initHash();
}

GBMMLOp::GBMMLOp(Tensor *A, Tensor *B, int dilation, Tensor *bias, ActType act)
    : GBMMLOp(A, B, new Tensor(), dilation, bias, act) {}

GBMMLOp::GBMMLOp(int dilation, Tensor *bias, ActType act)
    : Operator(GBMML), dilation(dilation), bias(bias), act(act) {
    initHash();
}

G2BMMGBMMLArgs GBMMLOp::getArgs() const {
    if (inputs.size() < 2)
        return G2BMMGBMMLArgs{0, 0, 0, 0, dilation};
    const Dim &a = inputs[0]->getDims();
    return G2BMMGBMMLArgs{a[0], a[1], inputs[1]->getDims()[2], (a[2] - 1) / 2, dilation};
}

void GBMMLOp::initHash() {
    auto [b, m, k, w, d] = getArgs();
    hash = type;
    for (int v : {b, m, k, w, d})
        hash = hashAppend(hash, (uint64_t)(int64_t)v);
    hash = hashPack(hash);
}

bool GBMMLOp::checkValid(const TensorVec &ins) {
    const Tensor *A = ins[0], *B = ins[1];
    if (A->getType() == Tensor::Weight && B->getType() == Tensor::Weight)
        return false;
    const Dim &a = A->getDims(), &b = B->getDims();
    return a.size() == 3 && b.size() == 3 && a[0] == b[0] && a[1] == b[1] && a[2] % 2 == 1;
}

Dim GBMMLOp::computeShape() {
    Dim ret = {inputs[0]->getDims()[0], inputs[0]->getDims()[1], inputs[1]->getDims()[2]};
    outputs[0]->setDims(ret);
    outputs[0]->setType(Tensor::Input);
    return ret;
}

int GBMMLOp::launch(pet_hip_stream_t stream) {
    const Dim &a = inputs[0]->getDims();
    return pet_hip_gbmml_f32(inputs[0]->devicePtr(), inputs[1]->devicePtr(),
                             outputs[0]->devicePtr(), a[0], a[1], (a[2] - 1) / 2,
                             inputs[1]->getDims()[2], dilation, stream);
}

// As the reference times _sgbmml (src/Graph/operator.cc:1560-1596).
double GBMMLOp::perf(PerfEngine *pe, int rounds, int warmupRounds) {
    G2BMMGBMMLArgs args = getArgs();
    if (pe->checkOpPerf(GBMML, args))
        return pe->getOpPerf(GBMML, args);
    auto [b, m, n, w, d] = args;
    double ms = INFINITY;
    if (b > 0 && m > 0 && n > 0) {
        float *A = pe->getMatA((size_t)b * m * (2 * w + 1)), *B = pe->getMatB((size_t)b * m * n);
        float *C = pe->getMatC((size_t)b * m * n);
        if (A && B && C)
            ms = timeFn(
                [&](pet_hip_stream_t st) { return pet_hip_gbmml_f32(A, B, C, b, m, w, n, d, st); },
                rounds, warmupRounds);
    }
    pe->saveOpPerf(GBMML, args, (float)ms);
    return pe->getOpPerf(GBMML, args);
}

std::string GBMMLOp::toString() const {
    std::ostringstream os;
    os << "GBMML[" << hash << "](";
    if (inputs.size() == 2)
        os << dimToString(inputs[0]->getDims()) << "," << dimToString(inputs[1]->getDims()) << ",";
    os << "dilation=" << dilation << ",act=" << act;
    if (inputs.size() == 2)
        os << "," << tensorTag("A", inputs[0]) << "," << tensorTag("B", inputs[1]) << ","
           << tensorTag("C", outputs[0]);
    os << ")";
    return os.str();
}

// ---- point dependences ------------------------------------------------------------
// For one output point, the input points it is computed from; the reference
// reports the same ranges (src/Graph/operator.cc:664-698, 1852-1880,
// 2212-2303, 2600-2616, 3005-3023) and evaluates the point on the host, here
// the returned closure runs the whole operator on the device.
namespace {
using PointDeps = std::pair<std::vector<DimRange>, std::function<bool()>>;

// Handles the ranges that are not a single point. Returns true when `out`
// already holds the answer.
bool symbolicRange(Operator *op, const DimRange &dr, size_t nIn, PointDeps &out) {
    if (dr.notValid()) {
        out = {};
        return true;
    }
    if (dr.isEmpty()) {
        out = {std::vector<DimRange>(nIn, DimRange::getEmpty()), []() { return true; }};
        return true;
    }
    if (!dr.isSinglePos()) {
        out = {std::vector<DimRange>(nIn, DimRange::getAllPos()),
               [op]() { return op->compute() != nullptr; }};
        return true;
    }
    return false;
}

bool insideDims(const Dim &pos, const Dim &dims) {
    if (pos.size() != dims.size())
        return false;
    for (size_t i = 0; i < pos.size(); ++i)
        if (pos[i] < 0 || pos[i] >= dims[i])
            return false;
    return true;
}
} // namespace

PointDeps MatmulOp::compute(DimRange dr) {
    PointDeps ret;
    if (symbolicRange(this, dr, inputs.size(), ret))
        return ret;
    const Dim &pos = dr.getBegin();
    if (pos.size() != 3 || !insideDims(pos, outputs[0]->getDims()))
        return {};
    int b = pos[0], m = pos[1], n = pos[2];
    int k = inputs[0]->getDims()[transA ? 1 : 2];
    DimRange lhs = transA ? DimRange({b, 0, m}, {b, k - 1, m}) : DimRange({b, m, 0}, {b, m, k - 1});
    DimRange rhs = transB ? DimRange({b, n, 0}, {b, n, k - 1}) : DimRange({b, 0, n}, {b, k - 1, n});
    return {{lhs, rhs}, [this]() { return compute() != nullptr; }};
}

PointDeps ConcatOp::compute(DimRange dr) {
    PointDeps ret;
    if (symbolicRange(this, dr, inputs.size(), ret))
        return ret;
    Dim src = dr.getBegin();
    if (!insideDims(src, outputs[0]->getDims()))
        return {};
    size_t which = 0;
    while (which < inputs.size() && src[dim] >= inputs[which]->getDims()[dim])
        src[dim] -= inputs[which++]->getDims()[dim];
    std::vector<DimRange> deps(inputs.size(), DimRange::getEmpty());
    deps[which] = DimRange(src);
    return {deps, [this]() { return compute() != nullptr; }};
}

PointDeps ExtendOp::compute(DimRange dr) {
    PointDeps ret;
    if (symbolicRange(this, dr, inputs.size(), ret))
        return ret;
    Dim src = dr.getBegin();
    if (!insideDims(src, outputs[0]->getDims()))
        return {};
    src[dim] %= inputs[0]->getDims()[dim];
    return {{DimRange(src)}, [this]() { return compute() != nullptr; }};
}

// Pow and BatchNorm read the input at the output's own position
// (src/Graph/operator.cc:3345-3357, 2683-2694).
PointDeps PowOp::compute(DimRange dr) {
    PointDeps ret;
    if (symbolicRange(this, dr, inputs.size(), ret))
        return ret;
    if (!insideDims(dr.getBegin(), outputs[0]->getDims()))
        return {};
    return {{DimRange(dr.getBegin())}, [this]() { return compute() != nullptr; }};
}

PointDeps BatchNormOp::compute(DimRange dr) {
    PointDeps ret;
    if (symbolicRange(this, dr, inputs.size(), ret))
        return ret;
    if (!insideDims(dr.getBegin(), outputs[0]->getDims()))
        return {};
    return {{DimRange(dr.getBegin())}, [this]() { return compute() != nullptr; }};
}

PointDeps EltwiseOp::compute(DimRange dr) {
    PointDeps ret;
    if (symbolicRange(this, dr, inputs.size(), ret))
        return ret;
    const Dim &pos = dr.getBegin();
    size_t flat = outputs[0]->getOffset(pos);
    if (flat == (size_t)-1)
        return {};
    std::vector<DimRange> deps;
    for (Tensor *in : inputs) // flat-modulo broadcast
        deps.emplace_back(cntToIdx(in->getDims(), flat % in->size()));
    return {deps, [this]() { return compute() != nullptr; }};
}

// y = x.reshape(flat).transpose(after).reshape(out): the output point's linear
// index over the permuted flat dims gives its flat coordinates; un-permuted,
// they give the linear index into the input. With boundary correction on, the
// dependence is reported as the whole input.
PointDeps TransposeOp::compute(DimRange dr) {
    PointDeps ret;
    if (symbolicRange(this, dr, inputs.size(), ret))
        return ret;
    auto whole = [this]() { return compute() != nullptr; };
    if (corrected())
        return {{DimRange::getAllPos()}, whole};
    Dim flat;
    size_t outOff = outputs[0]->getOffset(dr.getBegin());
    if (outOff == (size_t)-1 || !flatDims(flat))
        return {};
    std::vector<int> order = after.asVector();
    Dim permuted(order.size());
    for (size_t i = 0; i < order.size(); ++i)
        permuted[i] = flat[order[i]];
    Dim at = cntToIdx(permuted, outOff), src(flat.size(), 0);
    for (size_t i = 0; i < order.size(); ++i)
        src[order[i]] = at[i];
    size_t inOff = 0;
    for (size_t i = 0; i < flat.size(); ++i)
        inOff = inOff * (size_t)flat[i] + (size_t)src[i];
    return {{DimRange(cntToIdx(inputs[0]->getDims(), inOff))}, whole};
}

} // namespace tpm
