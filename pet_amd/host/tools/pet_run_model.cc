// Runs one of the benchmark networks through the host layer the way a PET user
// would: Graph -> SubGraph -> CodeEngine::instantiate (HIP graph) -> replay.
//
//   pet_run_model <dilated|dilated:pet|resnet18|bert|resnet3d18> [--rounds N] [--warmup N]
//                 [--check] [--tune] [--emit file.cpp]
// --tune: Operator::perf on every operator first (what the search does); convolutions then
// run with the algorithm that timed fastest for their arguments.
//
// Prints one JSON line: model, ms per replay, GFLOP, TFLOP/s, kernels in the
// captured graph, operators that cost no kernel (storage sharing, folded
// transposes). --check also runs the operators one by one (SubGraph::compute)
// and reports the largest difference between that result and the replayed graph's.
#include "code_engine.h"
#include "graph.h"
#include "models.h"

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>

using namespace tpm;

// Inputs and weights get uniform noise on the device, scaled so that activations
// keep their magnitude from layer to layer.
static bool fillInputs(SubGraph &sg, Graph &owner) {
    uint64_t seed = 1;
    auto fill = [&](Tensor *t, float lo, float hi) {
        float *p = t->devicePtr();
        if (!p || pet_hip_rand_uniform_f32(p, t->size(), seed++, lo, hi, petStream()) != PET_HIP_OK)
            return false;
        t->deviceWritten();
        t->setComputed();
        return true;
    };
    for (auto t : sg.getInputs()) {
        const Dim &d = t->getDims();
        size_t fanIn = 1;
        if (t->getType() == Tensor::Weight && d.size() >= 3) {
            if (d.size() == 3)
                fanIn = (size_t)d[1]; // [1, k, n]
            else
                for (size_t i = 1; i < d.size(); ++i)
                    fanIn *= (size_t)d[i];
        }
        float a = t->getType() == Tensor::Weight ? std::sqrt(3.0f / (float)fanIn) : 1.0f;
        if (t->size() == 1)
            a = 0.125f; // the attention scale
        if (!fill(t, t->size() == 1 ? a : -a, a))
            return false;
    }
    // bias / gamma / beta tensors hang off the operators, not the graph wiring
    for (auto t : owner.getTensors())
        if (t->getInputOf().empty() && t->getOutputOf() == nullptr && t->size() > 0 &&
            !t->getDims().empty())
            if (!fill(t, 0.9f, 1.1f))
                return false;
    return petOk(pet_hip_stream_sync(petStream()), "pet_hip_stream_sync");
}

int main(int argc, char **argv) {
    if (argc < 2) {
        std::fprintf(stderr, "usage: %s model [--rounds N] [--warmup N] [--check] [--tune] [--emit f]\n", argv[0]);
        return 2;
    }
    int rounds = 200, warmup = 20;
    bool check = false, tune = false;
    std::string emit;
    for (int i = 2; i < argc; ++i) {
        if (!std::strcmp(argv[i], "--rounds") && i + 1 < argc)
            rounds = std::atoi(argv[++i]);
        else if (!std::strcmp(argv[i], "--warmup") && i + 1 < argc)
            warmup = std::atoi(argv[++i]);
        else if (!std::strcmp(argv[i], "--check"))
            check = true;
        else if (!std::strcmp(argv[i], "--tune"))
            tune = true;
        else if (!std::strcmp(argv[i], "--emit") && i + 1 < argc)
            emit = argv[++i];
    }
    models::Model m;
    if (!models::byName(argv[1], m)) {
        std::fprintf(stderr, "unknown model %s\n", argv[1]);
        return 2;
    }
    if (!petInit()) {
        std::fprintf(stderr, "no gfx950 device: %s\n", pet_hip_last_error());
        return 3;
    }
    auto sg = std::make_shared<SubGraph>(m.graph->getOperators());
    if (!fillInputs(*sg, *m.graph))
        return 1;

    double maxDiff = -1.0, maxRef = 0.0;
    std::vector<float> eager;
    if (check) {
        if (!sg->compute())
            return 1;
        Tensor *o = sg->getOutputs()[0];
        const float *p = o->getDataPtr();
        eager.assign(p, p + o->size());
        sg->resetComputed();
    }
    CodeEngine ce;
    int tuned = 0;
    if (tune) {
        auto pe = std::make_shared<PerfEngine>();
        sg->perf(pe.get(), false);
        ce.importPerfEngine(pe);
        for (auto op : sg->getOperators())
            if (auto conv = dynamic_cast<ConvOp *>(op)) {
                tuned += conv->getAlgo() != 0;
                if (conv->getAlgo() != 0 && getenv("PET_HOST_TRACE"))
                    std::fprintf(stderr, "algo %d: %s\n", conv->getAlgo(), op->toString().c_str());
            }
            else if (auto c3 = dynamic_cast<Conv3dOp *>(op))
                tuned += c3->getAlgo() != 0;
            else if (auto mm = dynamic_cast<MatmulOp *>(op)) {
                tuned += mm->getAlgo() != 0;
                if (mm->getAlgo() != 0 && getenv("PET_HOST_TRACE"))
                    std::fprintf(stderr, "algo %d: %s\n", mm->getAlgo(), op->toString().c_str());
            }
    }
    auto exec = ce.instantiate(sg);
    if (!exec) {
        std::fprintf(stderr, "instantiate failed: %s\n", pet_hip_last_error());
        return 1;
    }
    if (!exec->launch() || !exec->sync())
        return 1;
    if (check) {
        Tensor *o = sg->getOutputs()[0];
        o->deviceWritten();
        const float *p = o->getDataPtr();
        maxDiff = 0.0;
        for (size_t i = 0; i < eager.size(); ++i) {
            if (!std::isfinite(p[i]))
                maxDiff = INFINITY;
            maxDiff = std::max(maxDiff, (double)std::fabs(p[i] - eager[i]));
            maxRef = std::max(maxRef, (double)std::fabs(eager[i]));
        }
    }
    double ms = exec->time(warmup, rounds);
    if (!emit.empty() && ce.genCode(sg, emit) != 0)
        return 1;
    std::printf("{\"model\": \"%s\", \"ms\": %.5f, \"gflop\": %.3f, \"tflops\": %.2f, "
                "\"operators\": %zu, \"kernels\": %zu, \"aliased\": %zu, \"folded\": %zu, "
                "\"hoisted_fills\": %zu",
                m.name.c_str(), ms, m.gflop, m.gflop / ms, sg->getOperators().size(),
                exec->numKernelOps(), exec->numAliasedOps(), exec->numFoldedOps(),
                exec->numHoistedFills());
    if (tune)
        std::printf(", \"off_default_algo\": %d", tuned);
    if (check)
        std::printf(", \"max_abs_diff_vs_eager\": %.3g, \"max_abs_eager\": %.3g", maxDiff, maxRef);
    std::printf("}\n");
    if (check && !(maxDiff <= 1e-4 * std::max(maxRef, 1e-30)))
        return 4;
    return 0;
}
