// Runs the reference's mutation generator (its own src/Mutant/generator.cc,
// built unchanged into libpet_refsearch.so) on this backend: one convolution
// goes in, the generator proposes transformed programs, each program is then
// executed on the device next to the original, compared element by element
// and timed through PerfEngine, which is what the reference's search does with
// a candidate (src/Graph/search_engine.cc:467-495).
//
//   pet_generator_driver n c h w f r pad dilation [min_exact]
//
// Exit status 0 when the generator produced candidates, every candidate ran, the
// best one agrees with the original on more than 70 % of the output (the
// generator's own acceptance threshold) and at least `min_exact` candidates
// agree everywhere. The generator accepts a candidate from eight sampled
// output points whose coordinates are all d/3 or 2d/3, so a candidate it
// accepts can still differ almost everywhere (two de-interleaves in a row fix
// exactly those rows of a 64-row image): the per-candidate fractions are
// reported, not required.
#include "generator.h"
#include "graph.h"
#include "operator.h"
#include "perf_engine.h"
#include "tensor.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <vector>

using namespace tpm;

static bool feedSameInputs(SubGraph *original, SubGraph *candidate) {
    std::map<uint64_t, Tensor *> byHash;
    for (auto t : original->getInputs())
        byHash[t->getHash()] = t;
    for (auto t : candidate->getInputs()) {
        auto it = byHash.find(t->getHash());
        if (it == byHash.end() || it->second->size() != t->size()) {
            std::printf("  input %lu of the candidate has no counterpart\n",
                        (unsigned long)t->getHash());
            return false;
        }
        t->setData(it->second->getDataPtr());
    }
    return true;
}

int main(int argc, char **argv) {
    if (argc < 9) {
        std::fprintf(stderr, "usage: %s n c h w f r pad dilation [min_exact]\n", argv[0]);
        return 2;
    }
    int n = atoi(argv[1]), c = atoi(argv[2]), h = atoi(argv[3]), w = atoi(argv[4]);
    int f = atoi(argv[5]), r = atoi(argv[6]), pad = atoi(argv[7]), dil = atoi(argv[8]);
    int minExact = argc > 9 ? atoi(argv[9]) : 0;

    Graph g;
    Tensor *x = g.tensor({n, c, h, w});
    Tensor *k = g.tensor({f, c, r, r});
    Operator *conv = g.conv(x, k, pad, pad, 1, 1, dil, dil);
    SubGraph original({conv});
    for (auto t : original.getTensors())
        t->dataMalloc();
    int seed = 1;
    for (auto t : original.getInputs())
        t->dataRand(seed++);

    Generator generator;
    std::vector<SubGraph *> candidates;
    generator.run(&original, candidates);
    std::printf("generator: %zu candidates for conv %dx%dx%dx%d * %dx%dx%dx%d pad %d dilation %d\n",
                candidates.size(), n, c, h, w, f, c, r, r, pad, dil);
    if (candidates.empty())
        return 1;

    // the generator re-seeded the inputs; compute the original once on them
    original.resetComputed();
    if (!original.compute())
        return 1;
    Tensor *want = original.getOutputs()[0];
    const VType *wantData = want->getDataPtr();

    PerfEngine pe;
    double baseMs = original.perf(&pe, false);
    std::printf("original: %.4f ms\n", baseMs);

    int exact = 0;
    bool ok = true;
    double bestFrac = 0.0;
    double bestMs = baseMs;
    int best = -1;
    for (size_t i = 0; i < candidates.size(); ++i) {
        SubGraph *cand = candidates[i];
        std::printf("candidate %zu:\n", i);
        for (auto op : cand->getOperators())
            std::printf("  %s\n", op->toString().c_str());
        if (!feedSameInputs(&original, cand)) {
            ok = false;
            continue;
        }
        cand->resetComputed();
        if (!cand->compute()) {
            std::printf("  did not run\n");
            ok = false;
            continue;
        }
        Tensor *got = nullptr;
        for (auto t : cand->getOutputs())
            if (!t->isNotCounted())
                got = t;
        if (got == nullptr || got->getDims() != want->getDims()) {
            std::printf("  output shape differs\n");
            ok = false;
            continue;
        }
        const VType *gotData = got->getDataPtr();
        size_t same = 0;
        for (size_t j = 0; j < want->size(); ++j)
            same += gotData[j] == wantData[j];
        double frac = (double)same / (double)want->size();
        double ms = cand->perf(&pe, false);
        std::printf("  equal on %.2f %% of the output, %.4f ms (original %.4f ms)\n", 100.0 * frac,
                    ms, baseMs);
        bestFrac = std::max(bestFrac, frac);
        if (same == want->size()) {
            ++exact;
            if (ms < bestMs) {
                bestMs = ms;
                best = (int)i;
            }
        }
    }
    std::printf("exact candidates: %d (need %d); fastest exact program: %s at %.4f ms\n", exact,
                minExact, best < 0 ? "the original" : ("candidate " + std::to_string(best)).c_str(),
                bestMs);
    std::fflush(stdout);
    // The generator and its scratch graph share operator ownership the way the
    // reference's do; leave their teardown to process exit.
    std::_Exit(ok && bestFrac > 0.7 && exact >= minExact ? 0 : 1);
}
