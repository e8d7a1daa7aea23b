// Runs the reference's search engine (its own src/Graph/search_engine.cc with its
// mutation generator, built unchanged into libpet_refsearch.so) on this backend:
// SearchEngine::run on one convolution, every candidate ranked by Operator::perf on the
// MI355X, then the chosen program is executed next to the original and compared.
//
//   pet_search_driver n c h w f r pad dilation [nnet]
//
// With "nnet" the mutation engine is the reference's NMutator (src/nnet/nmutator.cc)
// instead of its Generator. Its transforms leave MemBound placeholders without an
// expression for layout moves they only price; a best graph that holds one is costed but
// cannot be executed, and the comparison of outputs is left out for it.
//
// Prints what SearchEngine::run prints (its getPerf profile tables among it), the cost of
// the original and of bestGraph through SearchEngine::getPerf, and the agreement of the two
// programs. Exit status 0 when run() returned a graph, its cost is at most the original's,
// the profile total equals SubGraph::perf on the same PerfEngine memo, and the best program
// computes what the original computes.
#include "generator.h"
#include "graph.h"
#include "nnet/nmutator.h"
#include "operator.h"
#include "perf_engine.h"
#include "search_engine.h"
#include "tensor.h"

#include <cmath>
#include <csignal>
#include <cstdio>
#include <execinfo.h>
#include <unistd.h>
#include <cstdlib>
#include <map>
#include <string>

using namespace tpm;

// a crash inside the search prints where it happened before the process dies
static void onCrash(int sig) {
    void *frames[48];
    int n = backtrace(frames, 48);
    dprintf(2, "signal %d, backtrace:\n", sig);
    backtrace_symbols_fd(frames, n, 2);
    _exit(128 + sig);
}

int main(int argc, char **argv) {
    signal(SIGSEGV, onCrash);
    signal(SIGABRT, onCrash);
    if (argc < 9) {
        std::fprintf(stderr, "usage: %s n c h w f r pad dilation\n", argv[0]);
        return 2;
    }
    int n = atoi(argv[1]), c = atoi(argv[2]), h = atoi(argv[3]), w = atoi(argv[4]);
    int f = atoi(argv[5]), r = atoi(argv[6]), pad = atoi(argv[7]), dil = atoi(argv[8]);

    auto g = new Graph();
    Tensor *x = g->tensor({n, c, h, w});
    Tensor *k = g->tensor({f, c, r, r});
    g->conv(x, k, pad, pad, 1, 1, dil, dil);
    g->updateConnection();
    auto graph = std::make_shared<SubGraph>(g->getOperators());

    const bool useNnet = argc > 9 && std::string(argv[9]) == "nnet";
    std::shared_ptr<Mutator> mutator;
    if (useNnet)
        mutator = std::make_shared<NMutator>();
    else
        mutator = std::make_shared<Generator>();
    SearchEngine engine(mutator);
    std::shared_ptr<SubGraph> best;
    int err = engine.run(graph, best);
    std::fflush(stdout);
    if (err || !best) {
        std::printf("SearchEngine::run failed (%d)\n", err);
        std::_Exit(1);
    }
    double origin = engine.getPerf(graph, false, false);
    double chosen = engine.getPerf(best, false, false);
    std::printf("driver: original %.5f ms, bestGraph %.5f ms (%zu operators):\n", origin, chosen,
                best->getOperators().size());
    for (auto op : best->getOperators())
        std::printf("  %s\n", op->toString().c_str());
    bool ok = std::isfinite(origin) && std::isfinite(chosen) && chosen <= origin * 1.0001;

    // the profile of getPerf is the sum of Operator::perf, i.e. SubGraph::perf
    PerfEngine pe;
    double viaGraph = best->perf(&pe, false);
    std::printf("driver: SubGraph::perf of bestGraph on a fresh PerfEngine: %.5f ms\n", viaGraph);
    ok = ok && std::isfinite(viaGraph) && viaGraph > 0 &&
         std::fabs(viaGraph - chosen) <= 0.5 * std::max(viaGraph, chosen);

    bool runnable = true;
    for (auto op : best->getOperators())
        if (auto mb = dynamic_cast<MemBoundOp *>(op))
            runnable = runnable && mb->getExpr() != nullptr;
    if (!runnable) {
        std::printf("driver: bestGraph holds priced-only MemBound placeholders: not executed\n");
        std::printf("driver: %s\n", ok ? "ok" : "FAILED");
        std::fflush(stdout);
        std::_Exit(ok ? 0 : 1);
    }
    // run both programs on the same inputs
    int seed = 1;
    std::map<uint64_t, Tensor *> byHash;
    for (auto t : graph->getInputs()) {
        t->dataRand(seed++);
        byHash[t->getHash()] = t;
    }
    for (auto t : best->getInputs()) {
        auto it = byHash.find(t->getHash());
        if (it == byHash.end() || it->second->size() != t->size()) {
            std::printf("driver: input %lu of bestGraph has no counterpart\n",
                        (unsigned long)t->getHash());
            ok = false;
            continue;
        }
        t->setData(it->second->getDataPtr());
    }
    if (ok && graph->compute() && best->compute()) {
        Tensor *want = graph->getOutputs()[0], *got = nullptr;
        for (auto t : best->getOutputs())
            if (!t->isNotCounted())
                got = t;
        if (!got || got->size() != want->size()) {
            std::printf("driver: output sizes differ\n");
            ok = false;
        } else {
            size_t same = 0;
            const VType *a = want->getDataPtr(), *b = got->getDataPtr();
            for (size_t i = 0; i < want->size(); ++i)
                same += a[i] == b[i];
            std::printf("driver: bestGraph equals the original on %.2f %% of the output\n",
                        100.0 * same / want->size());
            ok = ok && same == want->size();
        }
    } else {
        std::printf("driver: a program did not run\n");
        ok = false;
    }
    std::printf("driver: %s\n", ok ? "ok" : "FAILED");
    std::fflush(stdout);
    // ownership of cloned operators is shared the way the reference shares it: no teardown
    std::_Exit(ok ? 0 : 1);
}
