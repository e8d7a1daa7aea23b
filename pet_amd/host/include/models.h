// The benchmark networks as tpm::Graph programs, built with the same Graph
// calls the reference's ONNX importer makes (python/cpp_plugin/import_onnx.py
// maps one ONNX node to one Graph builder): the dilated-convolution block as
// written and after PET's space-to-batch rewrite, ResNet-18, a BERT-base-shaped
// encoder and ResNet3D-18, all batch 1, BatchNorm folded into convolution bias.
#pragma once
#include "graph.h"
#include <memory>
#include <string>
#include <vector>

namespace tpm {
namespace models {

struct Model {
    std::string name;
    std::unique_ptr<Graph> graph; // owns operators and tensors (bias tensors included)
    double gflop = 0.0;           // convolutions and matmuls only, 2 * MACs
};

// Six 3x3 convolutions channels[0] -> ... -> channels.back() on 1 x c x hw x hw
// with dilation = padding = d and ReLU. spaceToBatch: the rows and columns are
// de-interleaved into the batch (two transposes), the convolutions run dense
// with padding 1, and two transposes interleave the result back
// (src/nnet/nmutator.cc:529-567 of the reference).
Model dilatedBlock(bool spaceToBatch, int hw = 64,
                   std::vector<int> channels = {512, 512, 512, 512, 256, 128, 64}, int d = 2);
Model resnet18(int hw = 224, int width = 64, int classes = 1000, bool mergedShortcut = false);
Model bertBase(int layers = 12, int seq = 128, int hidden = 768, int heads = 12, int ffn = 3072,
               bool mergedQkv = false);
Model resnet3d18(int t = 16, int hw = 112, int width = 64, int classes = 400);

// By name: "dilated", "dilated:pet", "resnet18", "bert", "resnet3d18".
bool byName(const std::string &name, Model &out);

} // namespace models
} // namespace tpm
