#include "models.h"

#include <cmath>

namespace tpm {
namespace models {

namespace {

struct Builder {
    Graph &g;
    double macs = 0.0;

    Tensor *fresh() { return g.tensor({}); }

    Tensor *conv(Tensor *x, int f, int k, int stride, int pad, int dil, bool relu, bool bias = true) {
        const Dim &d = x->getDims();
        Tensor *w = g.tensor({f, d[1], k, k});
        Tensor *b = bias ? g.tensor({f}) : nullptr;
        auto op = static_cast<ConvOp *>(g.conv(x, w, pad, pad, stride, stride, dil, dil, b));
        if (relu)
            op->setAct(Operator::Relu);
        Tensor *y = op->getOutputs()[0];
        macs += (double)y->size() * d[1] * k * k;
        return y;
    }

    Tensor *conv3d(Tensor *x, int f, Dim k, Dim stride, Dim pad, bool relu) {
        const Dim &d = x->getDims();
        Tensor *w = g.tensor({f, d[1], k[0], k[1], k[2]});
        Tensor *b = g.tensor({f});
        auto op = static_cast<Conv3dOp *>(g.conv3d(x, w, fresh(), pad, stride, {1, 1, 1}, b));
        if (relu)
            op->setAct(Operator::Relu);
        Tensor *y = op->getOutputs()[0];
        macs += (double)y->size() * d[1] * k[0] * k[1] * k[2];
        return y;
    }

    Tensor *linear(Tensor *x, int n, Operator::ActType act = Operator::None) { // x: [1, m, k]
        const Dim &d = x->getDims();
        Tensor *w = g.tensor({1, d[2], n});
        w->setType(Tensor::Weight);
        auto op = static_cast<MatmulOp *>(g.matmul(x, w, false, false, g.tensor({n})));
        op->setAct(act);
        macs += (double)d[1] * d[2] * n;
        return op->getOutputs()[0];
    }

    Tensor *bmm(Tensor *a, Tensor *b, bool transB) {
        const Dim &da = a->getDims(), &db = b->getDims();
        macs += (double)da[0] * da[1] * da[2] * (transB ? db[1] : db[2]);
        return g.matmul(a, b, false, transB)->getOutputs()[0];
    }

    Tensor *reshape(Tensor *x, const Dim &dims) {
        return g.reshape(x, g.tensor(dims))->getOutputs()[0];
    }
    Tensor *addRelu(Tensor *a, Tensor *b) {
        return g.relu(g.add({a, b})->getOutputs()[0])->getOutputs()[0];
    }
};

Model finish(const std::string &name, std::unique_ptr<Graph> g, double macs) {
    g->updateConnection();
    Model m;
    m.name = name;
    m.gflop = 2.0 * macs / 1e9;
    m.graph = std::move(g);
    return m;
}

} // namespace

Model dilatedBlock(bool spaceToBatch, int hw, std::vector<int> channels, int d) {
    std::unique_ptr<Graph> g(new Graph());
    Builder b{*g};
    Tensor *x = g->tensor({1, channels[0], hw, hw});
    if (!spaceToBatch) {
        for (size_t i = 1; i < channels.size(); ++i)
            x = b.conv(x, channels[i], 3, 1, d, d, true, false);
        return finish("dilated", std::move(g), b.macs);
    }
    // [N,C,H,W] -> [(d,N),C,H/d,W] -> [(d,d,N),C,H/d,W/d]; the runtime runs the two as one kernel
    x = g->transpose(x, 2, {{-1, 0}, 1, 2, 3}, d)->getOutputs()[0];
    x = g->transpose(x, 3, {{-1, 0}, 1, 2, 3}, d)->getOutputs()[0];
    for (size_t i = 1; i < channels.size(); ++i)
        x = b.conv(x, channels[i], 3, 1, 1, 1, true, false);
    // and back: the batch phase goes to the columns, then to the rows
    x = g->transpose(x, 0, {-1, 1, 2, {3, 0}}, -d)->getOutputs()[0];
    x = g->transpose(x, 0, {-1, 1, {2, 0}, 3}, -d)->getOutputs()[0];
    return finish("dilated:pet", std::move(g), b.macs);
}

Model resnet18(int hw, int width, int classes, bool mergedShortcut) {
    std::unique_ptr<Graph> g(new Graph());
    Builder b{*g};
    Tensor *x = g->tensor({1, 3, hw, hw});
    x = b.conv(x, width, 7, 2, 3, 1, true);
    x = g->maxpool(x, b.fresh(), 3, 3, 1, 1, 1, 1, 2, 2)->getOutputs()[0];
    for (int stage = 0; stage < 4; ++stage) {
        int cout = width << stage;
        for (int block = 0; block < 2; ++block) {
            int stride = (block == 0 && stage > 0) ? 2 : 1;
            Tensor *y, *skip;
            if (stride == 2 && mergedShortcut) {
                // PET's merge of two convolutions that read the same tensor
                // (src/Mutant/generator.cc:1236-1381): the 1x1 shortcut's filters are padded
                // to 3x3 and stacked under the first convolution's (weight-side work), one
                // convolution computes both, Split on the channel dim hands them out. The
                // ReLU belongs to the first half only and moves behind the Split.
                const double before = b.macs;
                Tensor *both = b.conv(x, 2 * cout, 3, 2, 1, 1, false);
                b.macs = before + (double)both->size() / 2 * x->getDims()[1] * (9 + 1); // nominal work
                const TensorVec &parts = g->split(both, 1, 2)->getOutputs();
                y = g->relu(parts[0])->getOutputs()[0];
                skip = parts[1];
            } else {
                y = b.conv(x, cout, 3, stride, 1, 1, true);
                skip = stride == 2 ? b.conv(x, cout, 1, 2, 0, 1, false) : x;
            }
            y = b.conv(y, cout, 3, 1, 1, 1, false);
            x = b.addRelu(y, skip);
        }
    }
    int c = x->getDims()[1];
    x = g->avgpool(x, b.fresh())->getOutputs()[0];
    x = b.linear(b.reshape(x, {1, 1, c}), classes);
    return finish(mergedShortcut ? "resnet18:pet" : "resnet18", std::move(g), b.macs);
}

Model bertBase(int layers, int seq, int hidden, int heads, int ffn, bool mergedQkv) {
    std::unique_ptr<Graph> g(new Graph());
    Builder b{*g};
    const int dh = hidden / heads;
    Tensor *x = g->tensor({1, seq, hidden});
    Tensor *scale = g->tensor({1}); // 1 / sqrt(dh), broadcast over the scores
    scale->setType(Tensor::Weight);
    auto toHeads = [&](Tensor *t) { // [1, seq, hidden] -> [heads, seq, dh]
        return g->transpose(b.reshape(t, {seq, hidden}), 1, {1, 0, -1}, dh)->getOutputs()[0];
    };
    auto norm = [&](Tensor *t) {
        return g->layernorm(t, b.fresh(), g->tensor({hidden}), g->tensor({hidden}))->getOutputs()[0];
    };
    for (int l = 0; l < layers; ++l) {
        Tensor *q, *k, *v;
        if (mergedQkv) {
            // PET's batch-matmul merge (src/Mutant/generator.cc:1495-1552) of the three
            // projections of x: lhs stacked on dim 0 (the same tensor three times), the
            // weights and biases stacked the same way, one Matmul with b = 3, Split on dim 0
            Tensor *x3 = g->concat({x, x, x}, 0)->getOutputs()[0];
            Tensor *w3 = g->tensor({3, hidden, hidden});
            w3->setType(Tensor::Weight);
            Tensor *y3 = g->matmul(x3, w3, false, false, g->tensor({3, hidden}))->getOutputs()[0];
            b.macs += 3.0 * seq * hidden * hidden;
            const TensorVec &parts = g->split(y3, 0, 3)->getOutputs();
            q = toHeads(parts[0]), k = toHeads(parts[1]), v = toHeads(parts[2]);
        } else {
            q = toHeads(b.linear(x, hidden)), k = toHeads(b.linear(x, hidden));
            v = toHeads(b.linear(x, hidden));
        }
        Tensor *s = b.bmm(q, k, true); // [heads, seq, seq]
        s = g->softmax(g->mul({s, scale})->getOutputs()[0], b.fresh(), 2)->getOutputs()[0];
        Tensor *ctx = b.bmm(s, v, false); // [heads, seq, dh]
        ctx = b.reshape(g->transpose(ctx, -1, {1, 0, 2})->getOutputs()[0], {1, seq, hidden});
        x = norm(g->add({x, b.linear(ctx, hidden)})->getOutputs()[0]);
        Tensor *h = b.linear(b.linear(x, ffn, Operator::Gelu), hidden);
        x = norm(g->add({x, h})->getOutputs()[0]);
    }
    return finish(mergedQkv ? "bert:pet" : "bert", std::move(g), b.macs);
}

Model resnet3d18(int t, int hw, int width, int classes) {
    std::unique_ptr<Graph> g(new Graph());
    Builder b{*g};
    Tensor *x = g->tensor({1, 3, t, hw, hw});
    x = b.conv3d(x, width, {3, 7, 7}, {1, 2, 2}, {1, 3, 3}, true);
    for (int stage = 0; stage < 4; ++stage) {
        int cout = width << stage;
        for (int block = 0; block < 2; ++block) {
            bool down = block == 0 && stage > 0;
            Dim stride = down ? Dim{2, 2, 2} : Dim{1, 1, 1};
            Tensor *y = b.conv3d(x, cout, {3, 3, 3}, stride, {1, 1, 1}, true);
            Tensor *skip = down ? b.conv3d(x, cout, {1, 1, 1}, {2, 2, 2}, {0, 0, 0}, false) : x;
            y = b.conv3d(y, cout, {3, 3, 3}, {1, 1, 1}, {1, 1, 1}, false);
            x = b.addRelu(y, skip);
        }
    }
    const Dim d = x->getDims(); // [1, c, t', h', w']
    x = b.reshape(x, {1, d[1], d[2], d[3] * d[4]});
    x = g->avgpool(x, b.fresh(), d[2], d[3] * d[4], 0, 0, 1, 1)->getOutputs()[0];
    x = b.linear(b.reshape(x, {1, 1, d[1]}), classes);
    return finish("resnet3d18", std::move(g), b.macs);
}

bool byName(const std::string &name, Model &out) {
    if (name == "dilated")
        out = dilatedBlock(false);
    else if (name == "dilated:pet")
        out = dilatedBlock(true);
    else if (name == "resnet18")
        out = resnet18();
    else if (name == "resnet18:pet")
        out = resnet18(224, 64, 1000, true);
    else if (name == "bert")
        out = bertBase();
    else if (name == "bert:pet")
        out = bertBase(12, 128, 768, 12, 3072, true);
    else if (name == "resnet3d18")
        out = resnet3d18();
    else
        return false;
    return true;
}

} // namespace models
} // namespace tpm
