// Drives GraphBase::importOnnx (pet_amd/host/src/onnx_import.cc) for the tests:
//   onnx_driver <model.onnx>                      prints the operators and the shapes of their
//                                                 outputs; no device needed
//   onnx_driver <model.onnx> <in.bin> <out.bin>   also feeds the graph's one non-weight input
//                                                 from raw float32, runs the graph on the
//                                                 device (SubGraph::compute) and writes its
//                                                 first output as raw float32
//   onnx_driver <model.onnx> --export <out.onnx>  also writes the imported graph back with
//                                                 GraphBase::exportOnnx (src/onnx_export.cc);
//                                                 no device needed
// Exit code 2: the importer refused the file; 3: the exporter refused the graph.
#include "graph.h"
#include "operator.h"
#include "tensor.h"

#include <cstdio>
#include <fstream>
#include <memory>
#include <string>
#include <vector>

using namespace tpm;

int main(int argc, char **argv) {
    if (argc != 2 && argc != 4) {
        std::fprintf(stderr, "usage: %s model.onnx [in.bin out.bin | --export out.onnx]\n", argv[0]);
        return 1;
    }
    auto g = std::make_unique<Graph>();
    if (!g->importOnnx(argv[1]))
        return 2;
    for (auto op : g->getOperators()) {
        std::printf("%s", op->toString().c_str());
        std::printf("  ->");
        for (auto t : op->getOutputs()) {
            std::printf(" [");
            const Dim &d = t->getDims();
            for (size_t i = 0; i < d.size(); ++i)
                std::printf("%s%d", i ? "," : "", d[i]);
            std::printf("]");
        }
        std::printf("\n");
    }
    std::printf("operators: %zu\n", g->getOperators().size());
    if (argc == 2)
        return 0;
    if (std::string(argv[2]) == "--export")
        return g->exportOnnx(argv[3]) ? 0 : 3;

    // the whole model on the device
    TensorVec feeds;
    for (auto t : g->getInputs())
        if (t->getType() != Tensor::Weight)
            feeds.push_back(t);
    if (feeds.size() != 1) {
        std::fprintf(stderr, "the driver feeds models with one input; this one has %zu\n",
                     feeds.size());
        return 1;
    }
    std::ifstream in(argv[2], std::ios::binary);
    std::vector<float> x(feeds[0]->size());
    in.read(reinterpret_cast<char *>(x.data()), (std::streamsize)(x.size() * sizeof(float)));
    if (!in) {
        std::fprintf(stderr, "%s holds fewer than %zu floats\n", argv[2], x.size());
        return 1;
    }
    // SubGraph clones tensors by hash without their data (as the reference's does): the
    // weights' values are handed over here; bias and batch-norm vectors are side pointers
    // of their operators and keep pointing at the Graph's tensors
    SubGraph sub(g->getOperators());
    Tensor *feed = nullptr;
    for (auto t : sub.getInputs()) {
        if (t->getHash() == feeds[0]->getHash())
            feed = t;
        for (auto src : g->getTensors())
            if (src->getType() == Tensor::Weight && src->getHash() == t->getHash())
                t->setData(src->getDataPtr());
    }
    if (!feed || !feed->setData(x.data())) {
        std::fprintf(stderr, "cannot feed the input\n");
        return 1;
    }
    if (!sub.compute()) {
        std::fprintf(stderr, "the graph did not run\n");
        return 1;
    }
    Tensor *out = sub.getOutputs().at(0);
    std::vector<float> y(out->size());
    for (size_t i = 0; i < y.size(); ++i)
        y[i] = out->getData(i);
    std::ofstream of(argv[3], std::ios::binary);
    of.write(reinterpret_cast<const char *>(y.data()), (std::streamsize)(y.size() * sizeof(float)));
    std::printf("output: %zu values\n", y.size());
    return 0;
}
