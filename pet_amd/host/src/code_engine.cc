#include "code_engine.h"

#include <algorithm>
#include <fstream>
#include <functional>
#include <map>
#include <set>
#include <sstream>
#include <unordered_map>

namespace tpm {

// ---- GraphExec ----------------------------------------------------------------

GraphExec::~GraphExec() {
    if (graph) {
        pet_hip_stream_sync(petStream());
        pet_hip_graph_destroy(graph);
    }
}

bool GraphExec::launch() {
    return graph && petOk(pet_hip_graph_launch(graph, petStream()), "pet_hip_graph_launch");
}

bool GraphExec::sync() { return petOk(pet_hip_stream_sync(petStream()), "pet_hip_stream_sync"); }

double GraphExec::time(int warmup, int rounds) {
    for (int i = 0; i < warmup; ++i)
        if (!launch())
            return INFINITY;
    pet_hip_event_t e0 = nullptr, e1 = nullptr;
    pet_hip_event_create(&e0);
    pet_hip_event_create(&e1);
    pet_hip_event_record(e0, petStream());
    for (int i = 0; i < rounds; ++i)
        launch();
    pet_hip_event_record(e1, petStream());
    pet_hip_event_sync(e1);
    float ms = 0.f;
    pet_hip_event_elapsed_ms(&ms, e0, e1);
    pet_hip_event_destroy(e0);
    pet_hip_event_destroy(e1);
    return rounds > 0 ? (double)ms / rounds : 0.0;
}

namespace {

// Which operators need no kernel because their tensors can share storage.
struct AliasPlan {
    std::set<const Operator *> skipped;
};

bool weightOnly(const Operator *op) {
    if (op->getInputs().empty())
        return false;
    for (auto t : op->getInputs())
        if (t->getType() != Tensor::Weight)
            return false;
    return true;
}

size_t elems(const Tensor *t) { return t->size(); }

// Transposes in a row become one kernel, as the reference's emitter collects a
// transpose whose only successor is a transpose into that successor
// (src/Graph/code_engine.cc:1428-1459): `folded` holds the operators that no
// longer run by themselves, `chains` maps the last transpose of a row to the
// whole row, first to last.
struct TransposeChains {
    std::set<const Operator *> folded;
    std::map<const Operator *, std::vector<TransposeOp *>> chains;
};

TransposeChains planTransposeChains(const OpVec &order, const TensorVec &graphOutputs,
                                    const std::set<const Operator *> &skipped) {
    TransposeChains plan;
    std::set<const Tensor *> outs(graphOutputs.begin(), graphOutputs.end());
    std::map<const Operator *, std::vector<TransposeOp *>> open; // keyed by current last op
    for (auto op : order) {
        auto tr = dynamic_cast<TransposeOp *>(op);
        if (!tr || skipped.count(op))
            continue;
        std::vector<TransposeOp *> row;
        Operator *prev = op->getInputs()[0]->getOutputOf();
        auto it = prev ? open.find(prev) : open.end();
        if (it != open.end()) {
            row = it->second;
            open.erase(it);
        }
        row.push_back(tr);
        Tensor *out = op->getOutputs()[0];
        const OpVec &users = out->getInputOf();
        bool continues = users.size() == 1 && dynamic_cast<TransposeOp *>(users[0]) != nullptr &&
                         !skipped.count(users[0]) && !outs.count(out) &&
                         weightOnly(op) == weightOnly(users[0]);
        if (continues) {
            open[op] = row;
        } else if (row.size() > 1) {
            for (size_t i = 0; i + 1 < row.size(); ++i)
                plan.folded.insert(row[i]);
            plan.chains[op] = row;
        }
    }
    return plan;
}

// "Contraction, Add with another tensor, activation" as one operator: the
// contraction's residual operand takes the other tensor and its epilogue the
// activation (cuDNN's fused convolution has the same z operand; the reference
// passes it with weight 0, src/Graph/code_engine.cc:955-977). The fused operator
// runs where the Add stood, when both of its inputs exist.
struct FusedTail {
    Operator *contraction = nullptr;
    Tensor *residual = nullptr;
    Operator::ActType act = Operator::None;
    Tensor *out = nullptr;
};

struct FusedTails {
    std::set<const Operator *> absorbed;          // contractions and activations that moved
    std::map<const Operator *, FusedTail> atAdd;  // keyed by the Add they run in place of
};

FusedTails planFusedTails(const OpVec &order, const TensorVec &graphOutputs,
                          const std::set<const Operator *> &skipped,
                          const std::function<bool(const FusedTail &)> &storageOk) {
    FusedTails plan;
    std::set<const Tensor *> outs(graphOutputs.begin(), graphOutputs.end());
    std::map<const Operator *, size_t> pos;
    for (size_t i = 0; i < order.size(); ++i)
        pos[order[i]] = i;
    // "contraction, activation": the activation rides in the contraction's epilogue (the
    // reference's fused cuDNN call, src/Graph/operator.cc:478-481). Keyed by the activation.
    for (auto op : order) {
        auto actOp = dynamic_cast<ActivationOp *>(op);
        if (actOp == nullptr || skipped.count(op))
            continue;
        Tensor *t = op->getInputs()[0];
        Operator *prod = t->getOutputOf();
        if (prod == nullptr || !prod->canTakeResidual() || skipped.count(prod) ||
            plan.absorbed.count(prod) || weightOnly(prod) || t->getInputOf().size() != 1 ||
            outs.count(t) || prod->getOutputs().size() != 1)
            continue;
        FusedTail tail;
        tail.contraction = prod;
        tail.residual = nullptr;
        tail.act = actOp->getActType();
        tail.out = actOp->getOutputs()[0];
        plan.absorbed.insert(prod);
        plan.atAdd[op] = tail;
    }
    for (auto op : order) {
        if (op->getType() != Operator::Add || op->getInputs().size() != 2 || skipped.count(op))
            continue;
        Tensor *sum = op->getOutputs()[0];
        Operator *pick = nullptr;
        Tensor *other = nullptr;
        for (int side = 0; side < 2; ++side) {
            Tensor *a = op->getInputs()[side], *b = op->getInputs()[1 - side];
            Operator *prod = a->getOutputOf();
            if (prod == nullptr || !prod->canTakeResidual() || skipped.count(prod) ||
                plan.absorbed.count(prod) || weightOnly(prod) || a == b ||
                a->getInputOf().size() != 1 || outs.count(a) || a->size() != sum->size() ||
                b->size() != sum->size() || prod->getOutputs().size() != 1)
                continue;
            if (pick == nullptr || pos[prod] > pos[pick]) { // the later one: its partner exists
                pick = prod;
                other = b;
            }
        }
        if (pick == nullptr)
            continue;
        FusedTail tail;
        tail.contraction = pick;
        tail.residual = other;
        tail.out = sum;
        const OpVec &users = sum->getInputOf();
        ActivationOp *actOp = nullptr;
        if (users.size() == 1 && !outs.count(sum) && !skipped.count(users[0]))
            actOp = dynamic_cast<ActivationOp *>(users[0]);
        if (actOp) {
            tail.act = actOp->getActType();
            tail.out = actOp->getOutputs()[0];
        }
        if (!storageOk(tail)) // residual and result share a buffer: keep the operators apart
            continue;
        if (actOp)
            plan.absorbed.insert(actOp);
        plan.absorbed.insert(pick);
        plan.atAdd[op] = tail;
    }
    return plan;
}

// What is fused across launches (pet_hip_call_flags):
//  * a contraction whose launch adds partial sums into its output starts by writing the
//    bias there; for the ones without a residual these initialisations are batched into
//    one launch at the start of the graph (nothing else writes those buffers);
//  * a convolution with ReLU whose result is only read by convolutions (as their input
//    or as the residual of their fused tail) may leave the ReLU to those readers, which
//    apply it on load: the activation launch that follows an accumulating launch
//    goes away. ReLU applied twice changes nothing, so the readers need not know
//    whether the producer accumulated.
struct FillSpec {
    Tensor *out, *bias;
    size_t outer, ch, inner;
};

struct LaunchPlan {
    std::map<const Operator *, unsigned> flags; // by contraction
    std::vector<FillSpec> fills;
    std::set<const Tensor *> preAct; // tensors that may hold values before their ReLU
};

bool isConvOp(const Operator *op) {
    return op->getType() == Operator::Conv || op->getType() == Operator::Conv3d;
}

bool isContraction(const Operator *op) { return isConvOp(op) || op->getType() == Operator::Matmul; }

Operator::ActType ownAct(Operator *op) {
    if (auto c = dynamic_cast<ConvOp *>(op))
        return c->getAct();
    if (auto c = dynamic_cast<Conv3dOp *>(op))
        return c->getAct();
    if (auto m = dynamic_cast<MatmulOp *>(op))
        return m->getAct();
    return Operator::None;
}

Tensor *ownBias(Operator *op) {
    if (auto c = dynamic_cast<ConvOp *>(op))
        return c->getBias();
    if (auto c = dynamic_cast<Conv3dOp *>(op))
        return c->getBias();
    if (auto m = dynamic_cast<MatmulOp *>(op))
        return m->getBias();
    return nullptr;
}

LaunchPlan planLaunchFlags(const OpVec &order, const TensorVec &graphOutputs,
                           const std::set<const Operator *> &skipped,
                           const std::set<const Operator *> &folded, const FusedTails &tails,
                           const std::function<bool(const Tensor *)> &ownStorage) {
    LaunchPlan plan;
    static const bool off = getenv("PET_HOST_NO_LAUNCH_FUSION") != nullptr;
    if (off)
        return plan;
    std::set<const Tensor *> outs(graphOutputs.begin(), graphOutputs.end());
    struct Eff {
        Operator *c;
        Tensor *out;
        Operator::ActType act;
        bool hasRes;
    };
    std::vector<Eff> effs;
    for (auto op : order) {
        if (skipped.count(op) || folded.count(op) || weightOnly(op))
            continue;
        auto tail = tails.atAdd.find(op);
        if (tail != tails.atAdd.end())
            effs.push_back({tail->second.contraction, tail->second.out, tail->second.act,
                            tail->second.residual != nullptr});
        else if (isContraction(op) && !tails.absorbed.count(op))
            effs.push_back({op, op->getOutputs()[0], ownAct(op), false});
    }
    for (auto &e : effs) {
        // With a residual the library adds it along with the partial sums of the first K
        // share. That pays for the small 2-D layers and matmuls (ResNet-18 0.197 -> 0.189 ms,
        // BERT-base 1.009 -> 0.990 ms: one launch less per block), not for the 3-D layers,
        // whose tiles then end on a dependent load (ResNet3D-18 1.058 -> 1.070 ms).
        if ((e.hasRes && e.c->getType() == Operator::Conv3d) || !ownStorage(e.out) ||
            !e.c->accumulates())
            continue;
        const Dim &d = e.out->getDims();
        FillSpec f{e.out, ownBias(e.c), 0, 0, 0};
        if (isConvOp(e.c)) {
            f.outer = (size_t)d[0];
            f.ch = (size_t)d[1];
            f.inner = e.out->size() / (f.outer * f.ch);
        } else { // matmul: the bias runs along the last dim
            f.ch = (size_t)d.back();
            f.outer = e.out->size() / f.ch;
            f.inner = 1;
        }
        plan.fills.push_back(f);
        plan.flags[e.c] |= PET_HIP_CALL_Y_INITIALISED;
    }
    for (auto &e : effs) {
        if (!isConvOp(e.c) || e.act != Operator::Relu || outs.count(e.out) || !ownStorage(e.out))
            continue;
        const OpVec &users = e.out->getInputOf();
        std::map<const Operator *, unsigned> want;
        bool ok = !users.empty();
        for (auto u : users) {
            auto tail = tails.atAdd.find(u);
            if (skipped.count(u) || folded.count(u) || weightOnly(u)) {
                ok = false;
            } else if (isConvOp(u) && u->getInputs()[0] == e.out && u->getInputs()[1] != e.out) {
                want[u] |= PET_HIP_CALL_X_RELU;
            } else if (dynamic_cast<PoolOp *>(u) != nullptr && tail == tails.atAdd.end()) {
                want[u] |= PET_HIP_CALL_X_RELU; // pooling applies it on the way in
            } else if (tail != tails.atAdd.end() && tail->second.residual == e.out &&
                       isConvOp(tail->second.contraction) &&
                       tail->second.contraction->getInputs()[1] != e.out) {
                want[tail->second.contraction] |= PET_HIP_CALL_RES_RELU;
            } else {
                ok = false;
            }
        }
        if (!ok)
            continue;
        for (auto &w : want)
            plan.flags[w.first] |= w.second;
        plan.flags[e.c] |= PET_HIP_CALL_DEFER_RELU;
        plan.preAct.insert(e.out);
    }
    return plan;
}

// The attention core as one launch: head-split Transposes of Q, K and V, Matmul(transB),
// Mul by a one-element scale, Softmax over the last axis, Matmul with V and the head-merge
// Transpose run as pet_hip_attention_f32 in place of the head merge, reading the
// [seq, heads*dh] projections and writing the merged [seq, heads*dh] result; none of the
// tensors in between is materialised. Everything in between must be used by this chain only.
struct FusedAttention {
    Tensor *q = nullptr, *k = nullptr, *v = nullptr; // [seq, heads*dh]
    Tensor *scale = nullptr;                         // one element, or none
    Tensor *out = nullptr;                           // [seq, heads, dh]
    int heads = 0, seq = 0, dh = 0;
};

struct FusedAttentions {
    std::set<const Operator *> absorbed;
    std::map<const Operator *, FusedAttention> atMerge; // keyed by the head-merge transpose
};

bool swapsFirstTwoOfThree(TransposeOp *tr) {
    auto ba = tr->getBeforeAndAfter();
    return ba.second.asVector() == std::vector<int>{1, 0, 2} && tr->getPaddingSize().first == 0 &&
           tr->getPaddingSize().second == 0;
}

FusedAttentions planAttention(const OpVec &order, const TensorVec &graphOutputs,
                              const std::set<const Operator *> &skipped,
                              const TransposeChains &rows) {
    FusedAttentions plan;
    static const bool off = getenv("PET_HOST_NO_ATTENTION_FUSION") != nullptr;
    if (off)
        return plan;
    std::set<const Tensor *> outs(graphOutputs.begin(), graphOutputs.end());
    auto soleUser = [&](Tensor *t) -> Operator * {
        return t->getInputOf().size() == 1 && !outs.count(t) ? t->getInputOf()[0] : nullptr;
    };
    auto plainMatmul = [&](Operator *op, bool transB) -> MatmulOp * {
        auto mm = dynamic_cast<MatmulOp *>(op);
        if (!mm || skipped.count(op) || mm->getTransA() || mm->getTransB() != transB ||
            mm->getBias() || mm->getAct() != Operator::None)
            return nullptr;
        return mm;
    };
    // [seq, heads*dh] --split the columns by dh, heads to the front--> [heads, seq, dh]
    auto headSplit = [&](Tensor *t, int heads, int seq, int dh) -> Tensor * {
        auto tr = dynamic_cast<TransposeOp *>(t->getOutputOf());
        if (!tr || skipped.count(tr) || rows.folded.count(tr) || rows.chains.count(tr) ||
            soleUser(t) == nullptr || tr->getSplit() != 1 || tr->getFactor() != dh ||
            !swapsFirstTwoOfThree(tr))
            return nullptr;
        Tensor *src = tr->getInputs()[0];
        if (src->getDims() != Dim{seq, heads * dh})
            return nullptr;
        Operator *prod = src->getOutputOf();
        return prod && rows.folded.count(prod) ? nullptr : src;
    };
    for (auto op : order) {
        auto sm = dynamic_cast<SoftmaxOp *>(op);
        if (!sm || skipped.count(op))
            continue;
        Tensor *scores = op->getInputs()[0], *scale = nullptr;
        const Dim sd = scores->getDims();
        if (sd.size() != 3 || sd[1] != sd[2] || sm->getAxis() != 2 || soleUser(scores) != op)
            continue;
        Operator *mulOp = nullptr;
        if (scores->getOutputOf() && scores->getOutputOf()->getType() == Operator::Mul &&
            scores->getOutputOf()->getInputs().size() == 2 && !skipped.count(scores->getOutputOf())) {
            mulOp = scores->getOutputOf();
            Tensor *a = mulOp->getInputs()[0], *b = mulOp->getInputs()[1];
            if (b->size() == 1 && a->size() == scores->size())
                scale = b, scores = a;
            else if (a->size() == 1 && b->size() == scores->size())
                scale = a, scores = b;
            else
                continue;
            if (soleUser(scores) != mulOp)
                continue;
        }
        MatmulOp *m1 = plainMatmul(scores->getOutputOf(), true);
        Tensor *probs = op->getOutputs()[0];
        MatmulOp *m2 = plainMatmul(soleUser(probs), false);
        if (!m1 || !m2 || m2->getInputs()[0] != probs)
            continue;
        const int heads = sd[0], seq = sd[1];
        Tensor *qh = m1->getInputs()[0], *kh = m1->getInputs()[1], *vh = m2->getInputs()[1];
        if (qh->getDims().size() != 3 || qh == kh || qh == vh || kh == vh)
            continue;
        const int dh = qh->getDims()[2];
        if (qh->getDims() != Dim{heads, seq, dh} || kh->getDims() != qh->getDims() ||
            vh->getDims() != qh->getDims() || seq > 512 ||
            (dh != 32 && dh != 64 && dh != 96 && dh != 128))
            continue;
        FusedAttention f;
        f.q = headSplit(qh, heads, seq, dh);
        f.k = headSplit(kh, heads, seq, dh);
        f.v = headSplit(vh, heads, seq, dh);
        Tensor *ctx = m2->getOutputs()[0];
        auto merge = dynamic_cast<TransposeOp *>(soleUser(ctx));
        if (!f.q || !f.k || !f.v || !merge || skipped.count(merge) || rows.folded.count(merge) ||
            rows.chains.count(merge) || merge->getSplit() >= 0 || !swapsFirstTwoOfThree(merge))
            continue;
        f.scale = scale;
        f.out = merge->getOutputs()[0];
        f.heads = heads;
        f.seq = seq;
        f.dh = dh;
        for (Tensor *t : {qh, kh, vh})
            plan.absorbed.insert(t->getOutputOf());
        plan.absorbed.insert(m1);
        if (mulOp)
            plan.absorbed.insert(mulOp);
        plan.absorbed.insert(op);
        plan.absorbed.insert(m2);
        plan.atMerge[merge] = f;
    }
    return plan;
}

int launchAttention(const FusedAttention &f, pet_hip_stream_t s) {
    const int ld = f.heads * f.dh;
    return pet_hip_attention_f32(f.q->devicePtr(), f.k->devicePtr(), f.v->devicePtr(),
                                 f.out->devicePtr(), 1, f.heads, f.seq, f.dh, ld, ld, ld, ld, 0, 0,
                                 0, 0, 1.0f, f.scale ? f.scale->devicePtr() : nullptr, s);
}

// Micro-ops of a row of transposes, lowered on the first one's input.
bool lowerChain(const std::vector<TransposeOp *> &row, TransProgram &prog) {
    std::vector<std::shared_ptr<TransBasic>> all;
    for (auto tr : row)
        for (auto &m : tr->getTTParam())
            all.push_back(m);
    return TransposeEngine::getInstance().lower(all, row.front()->getInputs()[0]->getDims(), prog);
}

int launchChain(const std::vector<TransposeOp *> &row, pet_hip_stream_t s) {
    TransProgram prog;
    if (!lowerChain(row, prog))
        return PET_HIP_ERR_INVALID;
    int outDims[PET_HIP_MAX_RANK], outRank = 0;
    return pet_hip_trans_chain(row.front()->getInputs()[0]->devicePtr(),
                               row.back()->getOutputs()[0]->devicePtr(), prog.inDims.data(),
                               (int)prog.inDims.size(), prog.ops.data(), prog.nops,
                               prog.perms.data(), outDims, &outRank, s);
}

// ---- layout operators as the addressing of the convolution next to them ----------
//
// A row of Transposes without correction parameters only regroups and reorders extents: every
// dim of its output is a run of factors, each with a stride in the row's input and one in its
// output. When the row feeds one 2-D convolution and channel, height and width of the
// convolution's input are single factors, the convolution reads the row's input through those
// strides (pet_hip_conv2d_view_f32) and the row is never launched; likewise a row behind a
// convolution, read the other way round, gives the strides the convolution writes through.
// PET's space-to-batch / batch-to-space pair around dilated convolutions is the case in point.
struct ViewFactor {
    long long ext, in, out;
    int src; // dim of the row's input the factor is cut from
};

bool chainFactors(const TransProgram &prog, std::vector<std::vector<ViewFactor>> &dims) {
    const int rank = (int)prog.inDims.size();
    dims.assign(rank, {});
    long long stride = 1;
    for (int i = rank - 1; i >= 0; --i) {
        if (prog.inDims[i] <= 0)
            return false;
        dims[i].push_back({prog.inDims[i], stride, 0, i});
        stride *= prog.inDims[i];
    }
    size_t pp = 0;
    for (int o = 0; o < prog.nops; ++o) {
        const int *op = &prog.ops[6 * o];
        if (op[0] == 0) { // split of dim op[1] into (rest, op[2])
            if (op[3] != 0 || op[4] != 0)
                return false;
            std::vector<ViewFactor> &outer = dims[op[1]], inner;
            long long have = 1, need = op[2];
            for (auto &f : outer)
                have *= f.ext;
            if (need <= 0 || have % need != 0)
                return false;
            while (need > 1) {
                if (outer.empty())
                    return false;
                ViewFactor last = outer.back();
                if (last.ext <= need) {
                    if (need % last.ext != 0)
                        return false;
                    inner.insert(inner.begin(), last);
                    need /= last.ext;
                    outer.pop_back();
                } else {
                    if (last.ext % need != 0)
                        return false;
                    inner.insert(inner.begin(), {need, last.in, 0, last.src});
                    outer.back() = {last.ext / need, last.in * need, 0, last.src};
                    need = 1;
                }
            }
            dims.insert(dims.begin() + op[1] + 1, inner);
        } else if (op[0] == 1) {
            std::vector<std::vector<ViewFactor>> moved(dims.size());
            for (size_t i = 0; i < dims.size(); ++i)
                moved[i] = dims[prog.perms[pp + i]];
            pp += dims.size();
            dims.swap(moved);
        } else {
            if (op[2] != 0 || op[3] != 0 || op[1] + 1 >= (int)dims.size())
                return false;
            std::vector<ViewFactor> &head = dims[op[1]], &tail = dims[op[1] + 1];
            head.insert(head.end(), tail.begin(), tail.end());
            dims.erase(dims.begin() + op[1] + 1);
        }
    }
    stride = 1;
    for (int i = (int)dims.size() - 1; i >= 0; --i)
        for (int j = (int)dims[i].size() - 1; j >= 0; --j) {
            dims[i][j].out = stride;
            stride *= dims[i][j].ext;
        }
    for (auto &d : dims) // factors of extent 1 are never stepped along
        d.erase(std::remove_if(d.begin(), d.end(), [](const ViewFactor &f) { return f.ext == 1; }),
                d.end());
    return true;
}

// (batch factors outermost first, channel, height, width) -> the C structure; `use_out`
// picks the strides in the row's output instead of its input
bool makeView(const std::vector<ViewFactor> &n, const std::vector<ViewFactor> &c,
              const std::vector<ViewFactor> &h, const std::vector<ViewFactor> &w, bool use_out,
              pet_hip_conv_view &v) {
    if (n.size() > 3 || c.size() > 1 || h.size() > 1 || w.size() > 1)
        return false;
    auto st = [&](const ViewFactor &f) { return use_out ? f.out : f.in; };
    v.c_stride = c.empty() ? 0 : st(c[0]);
    v.h_stride = h.empty() ? 0 : st(h[0]);
    v.w_stride = w.empty() ? 0 : st(w[0]);
    v.n_extent[0] = v.n_extent[1] = 1;
    v.n_stride[0] = v.n_stride[1] = v.n_stride[2] = 0;
    // innermost first; the outermost factor takes the third place, whose extent is implied
    std::vector<ViewFactor> in(n.rbegin(), n.rend());
    if (!in.empty()) {
        v.n_stride[2] = st(in.back());
        in.pop_back();
    }
    for (size_t i = 0; i < in.size(); ++i) {
        v.n_extent[i] = (int)in[i].ext;
        v.n_stride[i] = st(in[i]);
    }
    return true;
}

struct ConvView {
    bool hasX = false, hasY = false;
    pet_hip_conv_view x, y;
    Tensor *src = nullptr; // what the convolution reads instead of its input
    Tensor *dst = nullptr; // what it writes instead of its output
};

struct ConvViews {
    std::map<const Operator *, ConvView> byConv;
    std::set<const Operator *> folded;    // Transposes that never launch
    std::set<const Tensor *> notThere;    // tensors that are never written
};

ConvViews planConvViews(const OpVec &order, const TensorVec &graphOutputs,
                        const std::set<const Operator *> &skipped, const TransposeChains &rows,
                        const std::set<const Operator *> &taken) {
    ConvViews plan;
    static const bool off = getenv("PET_HOST_NO_CONV_VIEWS") != nullptr ||
                            getenv("PET_HOST_NO_LAUNCH_FUSION") != nullptr;
    if (off)
        return plan;
    std::set<const Tensor *> outs(graphOutputs.begin(), graphOutputs.end());
    auto supported = [](ConvOp *conv) {
        auto d = conv->getInputs()[0]->getDims(), w = conv->getInputs()[1]->getDims();
        int yes = 0;
        if (w[1] <= 0 || d[1] % w[1] != 0)
            return false;
        return pet_hip_conv2d_view_supported(d[0], d[1], d[2], d[3], w[0], w[2], w[3],
                                             conv->getPh(), conv->getPw(), conv->getSh(),
                                             conv->getSw(), conv->getDh(), conv->getDw(),
                                             d[1] / w[1], &yes) == PET_HIP_OK &&
               yes != 0;
    };
    for (auto op : order) {
        auto last = dynamic_cast<TransposeOp *>(op);
        if (!last || skipped.count(op) || rows.folded.count(op) || taken.count(op) || weightOnly(op))
            continue;
        std::vector<TransposeOp *> row = {last};
        if (rows.chains.count(op))
            row = rows.chains.at(op);
        bool free = true;
        for (auto tr : row)
            free = free && !taken.count(tr) && !plan.folded.count(tr);
        TransProgram prog;
        std::vector<std::vector<ViewFactor>> dims;
        if (!free || !lowerChain(row, prog) || !chainFactors(prog, dims))
            continue;
        Tensor *in = row.front()->getInputs()[0], *out = last->getOutputs()[0];
        // in front of a convolution: the row's output is that convolution's input and nothing else
        const OpVec &users = out->getInputOf();
        auto reader = users.size() == 1 ? dynamic_cast<ConvOp *>(users[0]) : nullptr;
        if (reader && !outs.count(out) && reader->getInputs()[0] == out &&
            reader->getInputs()[1] != out && !skipped.count(reader) && !taken.count(reader) &&
            !plan.byConv[reader].hasX && dims.size() == 4 && supported(reader)) {
            ConvView &cv = plan.byConv[reader];
            if (makeView(dims[0], dims[1], dims[2], dims[3], false, cv.x)) {
                cv.hasX = true;
                cv.src = in;
                for (auto tr : row) {
                    plan.folded.insert(tr);
                    plan.notThere.insert(tr->getOutputs()[0]);
                }
                continue;
            }
        }
        // behind a convolution: the row's input is that convolution's output, read by the row only
        auto writer = dynamic_cast<ConvOp *>(in->getOutputOf());
        if (writer && !outs.count(in) && in->getInputOf().size() == 1 && !skipped.count(writer) &&
            !taken.count(writer) && !plan.byConv[writer].hasY && prog.inDims.size() == 4 &&
            supported(writer)) {
            std::vector<std::vector<ViewFactor>> bySrc(4);
            for (auto &d : dims)
                for (auto &f : d)
                    bySrc[f.src].push_back(f);
            for (auto &d : bySrc)
                std::sort(d.begin(), d.end(),
                          [](const ViewFactor &a, const ViewFactor &b) { return a.in > b.in; });
            ConvView &cv = plan.byConv[writer];
            if (makeView(bySrc[0], bySrc[1], bySrc[2], bySrc[3], true, cv.y)) {
                cv.hasY = true;
                cv.dst = out;
                plan.notThere.insert(in);
                for (auto tr : row) {
                    plan.folded.insert(tr);
                    if (tr != last)
                        plan.notThere.insert(tr->getOutputs()[0]);
                }
            }
        }
    }
    for (auto it = plan.byConv.begin(); it != plan.byConv.end();)
        it = (it->second.hasX || it->second.hasY) ? std::next(it) : plan.byConv.erase(it);
    return plan;
}

// A fill planned for the output of a convolution that writes through strides moves to the
// buffer it writes: dense, with the channel factor's stride as the run per channel.
void retargetFills(LaunchPlan &lp, const ConvViews &views) {
    for (auto &cvp : views.byConv) {
        const ConvView &cv = cvp.second;
        if (!cv.hasY)
            continue;
        Tensor *own = const_cast<Operator *>(cvp.first)->getOutputs()[0];
        for (auto &f : lp.fills)
            if (f.out == own) {
                f.out = cv.dst;
                f.inner = cv.y.c_stride > 0 ? (size_t)cv.y.c_stride : 1;
                f.outer = cv.dst->size() / (f.ch * f.inner);
            }
    }
}

} // namespace

// A Matmul whose lhs is one [1, m, k] tensor stacked b times on dim 0 (an Extend, or a Concat
// of the same tensor) and read by nothing else reads that tensor directly: the stacking
// operator is skipped and never launched. Returns the skipped operators.
static std::set<const Operator *> planSharedLhs(const OpVec &order, const TensorVec &graphOutputs) {
    std::set<const Operator *> skipped;
    for (auto op : order) {
        auto mm = dynamic_cast<MatmulOp *>(op);
        if (!mm)
            continue;
        mm->setSharedLhs(nullptr);
        if (mm->getTransA())
            continue;
        Tensor *A = mm->getInputs()[0];
        Operator *prod = A->getOutputOf();
        if (prod == nullptr || A->getInputOf().size() != 1 ||
            std::find(graphOutputs.begin(), graphOutputs.end(), A) != graphOutputs.end())
            continue;
        Tensor *src = nullptr;
        if (auto ex = dynamic_cast<ExtendOp *>(prod)) {
            if (ex->getDim() == 0)
                src = prod->getInputs()[0];
        } else if (auto cat = dynamic_cast<ConcatOp *>(prod)) {
            if (cat->getDim() == 0) {
                src = prod->getInputs()[0];
                for (auto in : prod->getInputs())
                    if (in != src)
                        src = nullptr;
            }
        }
        if (src == nullptr || A->getDims().size() != 3 || src->size() * A->getDims()[0] != A->size() ||
            src->size() != (size_t)A->getDims()[1] * A->getDims()[2])
            continue;
        mm->setSharedLhs(src);
        skipped.insert(prod);
    }
    return skipped;
}

// A Split along `dim` cuts a tensor into contiguous slabs when every dim before it has extent
// 1 (dim 0 always; the channel dim of a batch-1 NCHW tensor).
static bool splitsIntoSlabs(const Operator *op) {
    if (op->getType() != Operator::Split)
        return false;
    const int dim = static_cast<const SplitOp *>(op)->getDim();
    const Dim &d = op->getInputs()[0]->getDims();
    for (int i = 0; i < dim && i < (int)d.size(); ++i)
        if (d[i] != 1)
            return false;
    return true;
}

// A ReLU whose input does not come straight from a contraction (those ride in the
// contraction's epilogue, planFusedTails) and whose result only convolutions and poolings read
// as their input is left to those readers (PET_HIP_CALL_X_RELU): the activation does not run
// and its output shares its input's storage. PET's merge of a block's first convolution with
// its 1x1 shortcut produces this: Conv (both filter banks) -> Split -> ReLU on the first half.
struct ReluIntoReaders {
    std::set<const Operator *> folded;
    std::map<const Operator *, unsigned> flags;
};

static ReluIntoReaders planReluIntoReaders(const OpVec &order, const TensorVec &graphOutputs,
                                           const std::set<const Operator *> &skipped) {
    ReluIntoReaders plan;
    static const bool off = getenv("PET_HOST_NO_LAUNCH_FUSION") != nullptr;
    if (off)
        return plan;
    for (auto op : order) {
        auto act = dynamic_cast<ActivationOp *>(op);
        if (act == nullptr || act->getActType() != Operator::Relu || skipped.count(op) ||
            weightOnly(op))
            continue;
        Tensor *in = op->getInputs()[0], *out = op->getOutputs()[0];
        Operator *prod = in->getOutputOf();
        if (prod != nullptr && prod->canTakeResidual())
            continue;
        if (std::find(graphOutputs.begin(), graphOutputs.end(), out) != graphOutputs.end() ||
            out->getInputOf().empty())
            continue;
        bool ok = true;
        for (auto u : out->getInputOf()) {
            const bool conv = u->getType() == Operator::Conv || u->getType() == Operator::Conv3d;
            const bool pool = dynamic_cast<PoolOp *>(u) != nullptr;
            if (skipped.count(u) || weightOnly(u) || !(conv || pool) || u->getInputs()[0] != out ||
                (conv && u->getInputs()[1] == out))
                ok = false;
        }
        if (!ok)
            continue;
        plan.folded.insert(op);
        for (auto u : out->getInputOf())
            plan.flags[u] |= PET_HIP_CALL_X_RELU;
    }
    return plan;
}

// Storage sharing, decided before anything is captured:
//  * Split on dim 0 (or on a dim behind dims of extent 1 only): every output is a slab of
//    the input buffer.
//  * Concat on dim 0: every input that an operator of this graph produces (and
//    that is used nowhere else in a conflicting way) is produced directly
//    into its slab of the output buffer.
//  * Reshape: the output is the input buffer.
static AliasPlan planAliases(const OpVec &order, const std::set<const Operator *> &alreadySkipped) {
    AliasPlan plan;
    plan.skipped.insert(alreadySkipped.begin(), alreadySkipped.end());
    std::set<const Tensor *> aliased;
    // tensors whose buffer another tensor already points into: moving such a
    // buffer (into a concat's output) would leave those views on freed memory
    std::set<const Tensor *> bases;
    for (auto op : order) {
        if (splitsIntoSlabs(op)) {
            Tensor *in = op->getInputs()[0];
            bases.insert(in);
            float *base = in->devicePtr();
            size_t off = 0;
            for (auto out : op->getOutputs()) {
                out->aliasDevice(base + off);
                aliased.insert(out);
                off += elems(out);
            }
            plan.skipped.insert(op);
        } else if (op->getType() == Operator::Reshape) {
            Tensor *in = op->getInputs()[0], *out = op->getOutputs()[0];
            if (elems(in) == elems(out)) {
                bases.insert(in);
                out->aliasDevice(in->devicePtr());
                aliased.insert(out);
                plan.skipped.insert(op);
            }
        }
    }
    // Concat: the output buffer must exist before its producers' buffers are
    // redirected, and a part can only live in one place.
    for (auto op : order) {
        if (op->getType() != Operator::Concat || static_cast<ConcatOp *>(op)->getDim() != 0)
            continue;
        bool ok = true;
        std::set<const Tensor *> seen;
        for (auto in : op->getInputs()) {
            Operator *prod = in->getOutputOf();
            if (prod == nullptr || aliased.count(in) || bases.count(in) ||
                !seen.insert(in).second || plan.skipped.count(prod))
                ok = false;
        }
        if (!ok)
            continue;
        Tensor *out = op->getOutputs()[0];
        float *base = out->devicePtr();
        size_t off = 0;
        for (auto in : op->getInputs()) {
            in->aliasDevice(base + off);
            aliased.insert(in);
            off += elems(in);
        }
        plan.skipped.insert(op);
    }
    return plan;
}

// Convolutions take the algorithm an imported PerfEngine found fastest for their
// arguments (src/Graph/code_engine.cc:874-878 reads the cuDNN algorithm the same way).
void CodeEngine::importAlgos(const OpVec &order) {
    if (!perfEngine)
        return;
    for (auto op : order)
        if (auto conv = dynamic_cast<ConvOp *>(op)) {
            ConvArgs args = conv->getArgs(perfEngine->withPenalty());
            if (perfEngine->checkOpPerf(Operator::Conv, args))
                conv->setAlgo(perfEngine->getConvAlgo(args));
        } else if (auto mm = dynamic_cast<MatmulOp *>(op)) {
            MatmulArgs args = mm->getArgs();
            if (perfEngine->checkOpPerf(Operator::Matmul, args))
                mm->setAlgo(perfEngine->getMatmulAlgo(args));
        }
}

std::unique_ptr<GraphExec> CodeEngine::instantiate(std::shared_ptr<SubGraph> &graph) {
    if (!petInit())
        return nullptr;
    OpVec order;
    if (!graph->topoOrder(order)) {
        std::fprintf(stderr, "[pet] graph has a cycle\n");
        return nullptr;
    }
    // settle every buffer (allocation + upload of host-side data) before capture
    for (auto t : graph->getTensors())
        if (!t->isValid() || t->devicePtr() == nullptr)
            return nullptr;
    for (auto op : order) {
        if (auto conv = dynamic_cast<ConvOp *>(op))
            if (conv->getBias())
                conv->getBias()->devicePtr();
        if (auto mm = dynamic_cast<MatmulOp *>(op))
            if (mm->getBias())
                mm->getBias()->devicePtr();
        if (auto c3 = dynamic_cast<Conv3dOp *>(op))
            if (c3->getBias())
                c3->getBias()->devicePtr();
        if (auto ln = dynamic_cast<LayerNormOp *>(op))
            for (Tensor *t : {ln->getGamma(), ln->getBeta()})
                if (t)
                    t->devicePtr();
        if (auto bn = dynamic_cast<BatchNormOp *>(op))
            for (Tensor *t : {bn->getScale(), bn->getBias(), bn->getMean(), bn->getVar()})
                t->devicePtr();
    }
    importAlgos(order);
    const std::set<const Operator *> stacked = planSharedLhs(order, graph->getOutputs());
    AliasPlan plan = planAliases(order, stacked);
    TransposeChains rows = planTransposeChains(order, graph->getOutputs(), plan.skipped);
    FusedTails tails = planFusedTails(order, graph->getOutputs(), plan.skipped,
                                      [](const FusedTail &f) {
                                          return f.residual->devicePtr() != f.out->devicePtr();
                                      }); // asked for tails with a residual only
    FusedAttentions att = planAttention(order, graph->getOutputs(), plan.skipped, rows);
    ReluIntoReaders relus = planReluIntoReaders(order, graph->getOutputs(), plan.skipped);
    for (auto op : relus.folded) // the readers read the ReLU's input
        op->getOutputs()[0]->aliasDevice(op->getInputs()[0]->devicePtr());
    std::set<const Operator *> inert = rows.folded; // operators that do not launch by themselves
    inert.insert(att.absorbed.begin(), att.absorbed.end());
    inert.insert(relus.folded.begin(), relus.folded.end());
    LaunchPlan lp = planLaunchFlags(order, graph->getOutputs(), plan.skipped, inert, tails,
                                    [](const Tensor *) { return true; });
    for (auto &f : relus.flags)
        lp.flags[f.first] |= f.second;
    // what another plan already runs its own way
    std::set<const Operator *> taken(att.absorbed.begin(), att.absorbed.end());
    taken.insert(relus.folded.begin(), relus.folded.end());
    taken.insert(tails.absorbed.begin(), tails.absorbed.end());
    for (auto &t : tails.atAdd)
        taken.insert(t.second.contraction);
    ConvViews views = planConvViews(order, graph->getOutputs(), plan.skipped, rows, taken);
    retargetFills(lp, views);
    auto flagsOf = [&](const Operator *op) {
        auto it = lp.flags.find(op);
        return it == lp.flags.end() ? 0u : it->second;
    };
    auto launchOp = [&](Operator *op, pet_hip_stream_t st) -> int {
        auto fa = att.atMerge.find(op);
        if (fa != att.atMerge.end())
            return launchAttention(fa->second, st);
        auto cv = views.byConv.find(op);
        if (cv != views.byConv.end()) {
            const ConvView &v = cv->second;
            return static_cast<ConvOp *>(op)->launchView(
                st, (v.hasX ? v.src : op->getInputs()[0])->devicePtr(), v.hasX ? &v.x : nullptr,
                (v.hasY ? v.dst : op->getOutputs()[0])->devicePtr(), v.hasY ? &v.y : nullptr,
                flagsOf(op));
        }
        auto tail = tails.atAdd.find(op);
        if (tail != tails.atAdd.end()) {
            const FusedTail &f = tail->second;
            return f.contraction->launchFused(st, f.residual ? f.residual->devicePtr() : nullptr,
                                              f.act, f.out->devicePtr(), flagsOf(f.contraction));
        }
        if (flagsOf(op))
            return op->launchFused(st, nullptr, ownAct(op), op->getOutputs()[0]->devicePtr(),
                                   flagsOf(op));
        auto it = rows.chains.find(op);
        return it == rows.chains.end() ? op->launch(st) : launchChain(it->second, st);
    };

    std::unique_ptr<GraphExec> exec(new GraphExec());
    pet_hip_stream_t s = petStream();
    // operators that only touch weights run once, outside the replayed graph
    // (the reference's "Preprocess operators for weights" block,
    // src/Graph/code_engine.cc:183-190)
    for (auto op : order)
        if (weightOnly(op) && !plan.skipped.count(op) && !rows.folded.count(op)) {
            if (launchOp(op, s) != PET_HIP_OK)
                return nullptr;
            for (auto t : op->getOutputs())
                t->deviceWritten();
        }
    // constant 3-D filters get their kt-major copy here, once, for the same reason
    for (auto op : order)
        if (auto c3 = dynamic_cast<Conv3dOp *>(op))
            if (c3->getInputs()[1]->getType() == Tensor::Weight && !plan.skipped.count(op))
                c3->prepackFilters(s);
    if (!petOk(pet_hip_stream_sync(s), "pet_hip_stream_sync"))
        return nullptr;
    if (!petOk(pet_hip_graph_begin_capture(s), "pet_hip_graph_begin_capture"))
        return nullptr;
    bool ok = true;
    if (!lp.fills.empty()) {
        std::vector<pet_hip_fill> fills;
        for (auto &f : lp.fills)
            fills.push_back({f.out->devicePtr(), f.bias ? f.bias->devicePtr() : nullptr, f.outer,
                             f.ch, f.inner});
        ok = petOk(pet_hip_bias_fill_batch(fills.data(), (int)fills.size(), s),
                   "pet_hip_bias_fill_batch");
        exec->nHoistedFills = fills.size();
    }
    for (auto op : order) {
        if (!ok)
            break;
        if (plan.skipped.count(op)) {
            exec->nAliasOps++;
            continue;
        }
        if (weightOnly(op))
            continue;
        if (rows.folded.count(op) || tails.absorbed.count(op) || att.absorbed.count(op) ||
            relus.folded.count(op) || views.folded.count(op)) {
            exec->nFoldedOps++;
            continue;
        }
        if (launchOp(op, s) != PET_HIP_OK) {
            std::fprintf(stderr, "[pet] capture of %s failed: %s\n", op->toString().c_str(),
                         pet_hip_last_error());
            ok = false;
            break;
        }
        exec->nLaunchOps++;
    }
    pet_hip_graph_t g = nullptr;
    if (!petOk(pet_hip_graph_end_capture(s, &g), "pet_hip_graph_end_capture") || !ok) {
        if (g)
            pet_hip_graph_destroy(g);
        return nullptr;
    }
    exec->graph = g;
    for (auto t : graph->getTensors())
        if (t->getOutputOf() != nullptr && !rows.folded.count(t->getOutputOf())) {
            // what a fused tail absorbed is not materialised either, except its last tensor
            const Operator *prod = t->getOutputOf();
            bool inside = tails.absorbed.count(prod) && dynamic_cast<const ActivationOp *>(prod) == nullptr;
            auto tail = tails.atAdd.find(prod);
            if (tail != tails.atAdd.end() && tail->second.out != t)
                inside = true;
            if (inside || lp.preAct.count(t) || att.absorbed.count(prod) || stacked.count(prod) ||
                relus.folded.count(prod) || views.notThere.count(t))
                continue; // not there, or there without its ReLU
            t->deviceWritten();
            t->setComputed();
        }
    return exec;
}

// ---- emitted program ------------------------------------------------------------

namespace {

struct Emitter {
    std::ostringstream os;
    std::unordered_map<const Tensor *, std::string> names;
    int counter = 0;

    std::string name(const Tensor *t) {
        auto it = names.find(t);
        if (it != names.end())
            return it->second;
        std::string n = "t" + std::to_string(counter++);
        names.emplace(t, n);
        return n;
    }
    std::string ints(const std::vector<int> &v) {
        std::string s = "{";
        for (size_t i = 0; i < v.size(); ++i)
            s += (i ? ", " : "") + std::to_string(v[i]);
        return s + "}";
    }
    void line(const std::string &l) { os << l << "\n"; }
};

std::string nullable(Emitter &e, Tensor *t) { return t ? e.name(t) : std::string("nullptr"); }

} // namespace

std::string CodeEngine::genCode(std::shared_ptr<SubGraph> &graph) {
    OpVec order;
    if (!graph->topoOrder(order))
        return "";
    importAlgos(order);
    Emitter e;
    e.line("// Generated by tpm::CodeEngine for the MI355X backend.");
    e.line("// Build: hipcc -O2 prog.cpp -I<repo>/include -L<repo>/pet_amd/lib -lpet_hip "
           "-Wl,-rpath,<repo>/pet_amd/lib -o prog");
    e.line("#include <cstdio>");
    e.line("#include <cstdlib>");
    e.line("#include \"pet_hip.h\"");
    e.line("#define CHECK(x) do { int _s = (x); if (_s) { std::fprintf(stderr, \"%s: %s\\n\", #x, "
           "pet_hip_last_error()); std::exit(1); } } while (0)");
    e.line("int main() {");
    e.line("    CHECK(pet_hip_init(0));");
    e.line("    pet_hip_stream_t s; CHECK(pet_hip_stream_create(&s));");
    // tensors (bias side pointers included)
    std::vector<Tensor *> all(graph->getTensors().begin(), graph->getTensors().end());
    for (auto op : order) {
        if (auto conv = dynamic_cast<ConvOp *>(op))
            if (conv->getBias())
                all.push_back(conv->getBias());
        if (auto mm = dynamic_cast<MatmulOp *>(op))
            if (mm->getBias())
                all.push_back(mm->getBias());
        if (auto c3 = dynamic_cast<Conv3dOp *>(op))
            if (c3->getBias())
                all.push_back(c3->getBias());
        if (auto ln = dynamic_cast<LayerNormOp *>(op))
            for (Tensor *t : {ln->getGamma(), ln->getBeta()})
                if (t)
                    all.push_back(t);
        if (auto bn = dynamic_cast<BatchNormOp *>(op))
            for (Tensor *t : {bn->getScale(), bn->getBias(), bn->getMean(), bn->getVar()})
                all.push_back(t);
    }
    std::set<const Tensor *> viewOf, viewBase;
    // the buffer a view lives in (views of views resolve to the allocation at the bottom)
    std::map<const Tensor *, const Tensor *> bufferOf;
    auto buffer = [&](const Tensor *t) {
        auto it = bufferOf.find(t);
        return it == bufferOf.end() ? t : it->second;
    };
    std::set<const Operator *> skipped = planSharedLhs(order, graph->getOutputs());
    // storage sharing, mirrored from instantiate(): split / concat on dim 0, reshape
    std::vector<std::string> aliasLines;
    for (auto op : order) {
        if (splitsIntoSlabs(op)) {
            size_t off = 0;
            viewBase.insert(op->getInputs()[0]);
            for (auto out : op->getOutputs()) {
                aliasLines.push_back("    float *" + e.name(out) + " = " +
                                     e.name(op->getInputs()[0]) + " + " + std::to_string(off) + ";");
                viewOf.insert(out);
                bufferOf[out] = buffer(op->getInputs()[0]);
                off += out->size();
            }
            skipped.insert(op);
        } else if (op->getType() == Operator::Reshape) {
            aliasLines.push_back("    float *" + e.name(op->getOutputs()[0]) + " = " +
                                 e.name(op->getInputs()[0]) + ";");
            viewOf.insert(op->getOutputs()[0]);
            bufferOf[op->getOutputs()[0]] = buffer(op->getInputs()[0]);
            viewBase.insert(op->getInputs()[0]);
            skipped.insert(op);
        }
    }
    for (auto op : order) {
        if (op->getType() != Operator::Concat || static_cast<ConcatOp *>(op)->getDim() != 0)
            continue;
        bool ok = true;
        std::set<const Tensor *> seen;
        for (auto in : op->getInputs())
            if (in->getOutputOf() == nullptr || viewOf.count(in) || viewBase.count(in) ||
                !seen.insert(in).second ||
                skipped.count(in->getOutputOf()))
                ok = false;
        if (!ok)
            continue;
        size_t off = 0;
        for (auto in : op->getInputs()) {
            aliasLines.push_back("    float *" + e.name(in) + " = " + e.name(op->getOutputs()[0]) +
                                 " + " + std::to_string(off) + ";");
            viewOf.insert(in);
            bufferOf[in] = buffer(op->getOutputs()[0]);
            off += in->size();
        }
        skipped.insert(op);
    }
    // a ReLU left to the convolutions that read it: its output is its input
    ReluIntoReaders relus = planReluIntoReaders(order, graph->getOutputs(), skipped);
    for (auto op : order)
        if (relus.folded.count(op)) {
            aliasLines.push_back("    float *" + e.name(op->getOutputs()[0]) + " = " +
                                 e.name(op->getInputs()[0]) + ";");
            viewOf.insert(op->getOutputs()[0]);
            bufferOf[op->getOutputs()[0]] = buffer(op->getInputs()[0]);
            viewBase.insert(op->getInputs()[0]);
            skipped.insert(op);
        }
    TransposeChains rows = planTransposeChains(order, graph->getOutputs(), skipped);
    uint64_t seed = 1;
    for (auto t : all) {
        if (viewOf.count(t))
            continue;
        if (t->getOutputOf() != nullptr && rows.folded.count(t->getOutputOf()))
            continue; // inside a row of transposes: never materialised
        std::string n = e.name(t);
        e.line("    float *" + n + "; CHECK(pet_hip_malloc((void **)&" + n + ", " +
               std::to_string(std::max<size_t>(t->size(), 1)) + " * sizeof(float)));");
        // inputs and weights get uniform noise, as the reference's emitted
        // program does with cuRAND (src/Graph/code_engine.cc:582-583)
        if (t->getOutputOf() == nullptr)
            e.line("    CHECK(pet_hip_rand_uniform_f32(" + n + ", " + std::to_string(t->size()) +
                   ", " + std::to_string(seed++) + "ull, -1.f, 1.f, s));");
    }
    for (auto &l : aliasLines)
        e.line(l);

    std::map<const Operator *, std::string> packedName; // Conv3d -> its kt-major filter copy
    FusedTails tails = planFusedTails(order, graph->getOutputs(), skipped, [&](const FusedTail &f) {
        return buffer(f.residual) != buffer(f.out); // as instantiate(): different storage
    });
    FusedAttentions att = planAttention(order, graph->getOutputs(), skipped, rows);
    std::set<const Operator *> inert = rows.folded;
    inert.insert(att.absorbed.begin(), att.absorbed.end());
    LaunchPlan lp = planLaunchFlags(order, graph->getOutputs(), skipped, inert, tails,
                                    [](const Tensor *) { return true; });
    for (auto &f : relus.flags)
        lp.flags[f.first] |= f.second;
    std::set<const Operator *> taken(att.absorbed.begin(), att.absorbed.end()); // as instantiate()
    taken.insert(tails.absorbed.begin(), tails.absorbed.end());
    for (auto &t : tails.atAdd)
        taken.insert(t.second.contraction);
    ConvViews views = planConvViews(order, graph->getOutputs(), skipped, rows, taken);
    retargetFills(lp, views);
    auto flagsOf = [&](const Operator *op) {
        auto it = lp.flags.find(op);
        return it == lp.flags.end() ? 0u : it->second;
    };
    auto viewText = [](const pet_hip_conv_view &v) {
        std::ostringstream t;
        t << "{" << v.c_stride << ", " << v.h_stride << ", " << v.w_stride << ", {"
          << v.n_extent[0] << ", " << v.n_extent[1] << "}, {" << v.n_stride[0] << ", "
          << v.n_stride[1] << ", " << v.n_stride[2] << "}}";
        return t.str();
    };
    // set while a contraction is emitted in place of the Add that follows it
    const FusedTail *tail = nullptr;
    std::function<bool(Operator *)> emitOp = [&](Operator *op) -> bool {
        std::ostringstream c;
        auto in = [&](size_t i) { return e.name(op->getInputs()[i]); };
        auto out = [&](size_t i) {
            return tail ? e.name(tail->out) : e.name(op->getOutputs()[i]);
        };
        const std::string res =
            tail ? (tail->residual ? e.name(tail->residual) : std::string("nullptr")) + ", " : "";
        auto actOf = [&](Operator::ActType own) { return (int)(tail ? tail->act : own); };
        if (tails.atAdd.count(op) && tail == nullptr) {
            tail = &tails.atAdd.at(op);
            bool ok = emitOp(tail->contraction);
            tail = nullptr;
            return ok;
        }
        if (att.atMerge.count(op)) {
            const FusedAttention &f = att.atMerge.at(op);
            const int ld = f.heads * f.dh;
            c << "pet_hip_attention_f32(" << e.name(f.q) << ", " << e.name(f.k) << ", "
              << e.name(f.v) << ", " << e.name(f.out) << ", 1, " << f.heads << ", " << f.seq << ", "
              << f.dh << ", " << ld << ", " << ld << ", " << ld << ", " << ld
              << ", 0, 0, 0, 0, 1.0f, " << nullable(e, f.scale) << ", s)";
        } else if (views.byConv.count(op)) {
            // the Transposes next to this convolution are its addressing
            auto conv = static_cast<ConvOp *>(op);
            const ConvView &v = views.byConv.at(op);
            auto d = op->getInputs()[0]->getDims(), w = op->getInputs()[1]->getDims();
            const std::string id = std::to_string(op->getGuid());
            if (v.hasX)
                e.line("    static const pet_hip_conv_view xv" + id + " = " + viewText(v.x) + ";");
            if (v.hasY)
                e.line("    static const pet_hip_conv_view yv" + id + " = " + viewText(v.y) + ";");
            c << "pet_hip_conv2d_view_f32(" << (v.hasX ? e.name(v.src) : in(0)) << ", "
              << (v.hasX ? "&xv" + id : std::string("nullptr")) << ", " << in(1) << ", "
              << nullable(e, conv->getBias()) << ", nullptr, "
              << (v.hasY ? e.name(v.dst) : out(0)) << ", "
              << (v.hasY ? "&yv" + id : std::string("nullptr")) << ", " << d[0] << ", " << d[1]
              << ", " << d[2] << ", " << d[3] << ", " << w[0] << ", " << w[2] << ", " << w[3] << ", "
              << conv->getPh() << ", " << conv->getPw() << ", " << conv->getSh() << ", "
              << conv->getSw() << ", " << conv->getDh() << ", " << conv->getDw() << ", "
              << d[1] / w[1] << ", " << (int)conv->getAct() << ", "
              << (flagsOf(op) | PET_HIP_CONV_ALGO(conv->getAlgo())) << "u, s)";
        } else if (auto conv = dynamic_cast<ConvOp *>(op)) {
            auto d = op->getInputs()[0]->getDims(), w = op->getInputs()[1]->getDims();
            const unsigned fl = flagsOf(op) | PET_HIP_CONV_ALGO(conv->getAlgo());
            c << (fl     ? "pet_hip_conv2d_ex_f32("
                  : tail ? "pet_hip_conv2d_res_f32("
                         : "pet_hip_conv2d_f32(")
              << in(0) << ", " << in(1) << ", " << nullable(e, conv->getBias()) << ", "
              << (fl && !tail ? std::string("nullptr, ") : res) << out(0) << ", " << d[0] << ", "
              << d[1] << ", " << d[2] << ", " << d[3] << ", " << w[0] << ", " << w[2] << ", " << w[3]
              << ", " << conv->getPh() << ", " << conv->getPw() << ", " << conv->getSh() << ", "
              << conv->getSw() << ", " << conv->getDh() << ", " << conv->getDw() << ", "
              << d[1] / w[1] << ", " << actOf(conv->getAct()) << ", "
              << (fl ? std::to_string(fl) + "u, " : std::string()) << "s)";
        } else if (auto c3 = dynamic_cast<Conv3dOp *>(op)) {
            auto d = op->getInputs()[0]->getDims(), w = op->getInputs()[1]->getDims();
            // filters with a kt-major copy (made before capture, below) use it
            const bool pk = packedName.count(op) != 0;
            const std::string filt =
                pk ? packedName[op] + "_ok ? " + packedName[op] + " : " + in(1) : in(1);
            const unsigned fl = flagsOf(op);
            if (tail || fl)
                c << (fl ? "pet_hip_conv3d_ex_f32(" : "pet_hip_conv3d_res_f32(") << in(0) << ", "
                  << filt << ", " << (pk ? packedName[op] + "_ok" : std::string("0")) << ", ";
            else if (pk)
                c << "(" << packedName[op] << "_ok ? pet_hip_conv3d_packed_f32 : "
                  << "pet_hip_conv3d_f32)(" << in(0) << ", " << filt << ", ";
            else
                c << "pet_hip_conv3d_f32(" << in(0) << ", " << in(1) << ", ";
            c << nullable(e, c3->getBias()) << ", " << (fl && !tail ? std::string("nullptr, ") : res)
              << out(0);
            for (int v : {d[0], d[1], d[2], d[3], d[4], w[0], w[2], w[3], w[4]})
                c << ", " << v;
            for (const Dim *v : {&c3->getPad(), &c3->getStride(), &c3->getDilation()})
                for (int x : *v)
                    c << ", " << x;
            c << ", " << d[1] / w[1] << ", " << actOf(c3->getAct()) << ", "
              << (fl ? std::to_string(fl) + "u, " : std::string()) << "s)";
        } else if (auto ct = dynamic_cast<ConvTransOp *>(op)) {
            auto d = op->getInputs()[0]->getDims(), w = op->getInputs()[1]->getDims();
            c << "pet_hip_conv_trans_f32(" << in(0) << ", " << in(1) << ", "
              << nullable(e, ct->getBias()) << ", " << out(0);
            for (int v : {d[0], d[1], d[2], d[3], w[0], w[1], w[3], ct->getPh(), ct->getPw(),
                          ct->getSh(), ct->getSw(), ct->getDh(), ct->getDw(), ct->getOph(),
                          ct->getOpw(), (int)ct->getAct()})
                c << ", " << v;
            c << ", s)";
        } else if (auto g2 = dynamic_cast<G2BMMOp *>(op)) {
            auto d = op->getInputs()[0]->getDims();
            c << "pet_hip_g2bmm_f32(" << in(0) << ", " << in(1) << ", " << out(0) << ", " << d[0]
              << ", " << d[1] << ", " << d[2] << ", " << g2->getWidth() << ", "
              << g2->getDilation() << ", s)";
        } else if (auto gb = dynamic_cast<GBMMLOp *>(op)) {
            auto d = op->getInputs()[0]->getDims();
            c << "pet_hip_gbmml_f32(" << in(0) << ", " << in(1) << ", " << out(0) << ", " << d[0]
              << ", " << d[1] << ", " << (d[2] - 1) / 2 << ", " << op->getInputs()[1]->getDims()[2]
              << ", " << gb->getDilation() << ", s)";
        } else if (auto ln = dynamic_cast<LayerNormOp *>(op)) {
            size_t cols = (size_t)op->getInputs()[0]->getDims().back();
            c << "pet_hip_layernorm(" << in(0) << ", " << nullable(e, ln->getGamma()) << ", "
              << nullable(e, ln->getBeta()) << ", " << out(0) << ", "
              << op->getInputs()[0]->size() / cols << ", " << cols << ", " << ln->getEps()
              << "f, s)";
        } else if (auto mm = dynamic_cast<MatmulOp *>(op)) {
            bool ta, tb;
            int b, m, n, k;
            std::tie(ta, tb, b, m, n, k) = mm->getArgs();
            const unsigned fl = flagsOf(op) | mm->operandFlags() | PET_HIP_CONV_ALGO(mm->getAlgo());
            c << (fl     ? "pet_hip_bmm_ex_f32("
                  : tail ? "pet_hip_bmm_res_f32("
                         : "pet_hip_bmm_f32(")
              << ta << ", " << tb << ", " << b << ", " << m << ", " << n << ", " << k << ", "
              << (mm->getSharedLhs() ? e.name(mm->getSharedLhs()) : in(0)) << ", " << in(1) << ", " << out(0) << ", " << nullable(e, mm->getBias())
              << ", "
              << (tail ? res : fl ? std::string("nullptr, ") : std::string())
              << actOf(mm->getAct()) << ", " << (fl ? std::to_string(fl) + "u, " : std::string())
              << "s)";
        } else if (auto tr = dynamic_cast<TransposeOp *>(op)) {
            TransProgram prog;
            std::vector<TransposeOp *> row = {tr};
            if (rows.chains.count(op))
                row = rows.chains.at(op);
            if (!lowerChain(row, prog))
                return false;
            std::string id = std::to_string(op->getGuid());
            std::string src = e.name(row.front()->getInputs()[0]);
            e.line("    static const int tin" + id + "[] = " + e.ints(prog.inDims) + ", tops" + id +
                   "[] = " + e.ints(prog.ops) + ", tperm" + id + "[] = " + e.ints(prog.perms) + ";");
            e.line("    // " + TransposeEngine::getInstance().describe(prog));
            c << "pet_hip_trans_chain(" << src << ", " << out(0) << ", tin" << id << ", "
              << prog.inDims.size() << ", tops" << id << ", " << prog.nops << ", tperm" << id
              << ", odims, &orank, s)";
        } else if (auto sp = dynamic_cast<SplitOp *>(op)) {
            std::string id = std::to_string(op->getGuid());
            std::string ptrs = "{";
            std::vector<int> sizes;
            for (size_t i = 0; i < op->getOutputs().size(); ++i) {
                ptrs += (i ? ", " : "") + out(i);
                sizes.push_back(op->getOutputs()[i]->getDims()[sp->getDim()]);
            }
            e.line("    float *souts" + id + "[] = " + ptrs + "}; static const int sdims" + id +
                   "[] = " + e.ints(op->getInputs()[0]->getDims()) + ", ssz" + id +
                   "[] = " + e.ints(sizes) + ";");
            c << "pet_hip_split(" << in(0) << ", souts" << id << ", " << sizes.size() << ", sdims"
              << id << ", " << op->getInputs()[0]->getDims().size() << ", " << sp->getDim()
              << ", ssz" << id << ", s)";
        } else if (auto cc = dynamic_cast<ConcatOp *>(op)) {
            std::string id = std::to_string(op->getGuid());
            std::string ptrs = "{";
            std::vector<int> sizes;
            for (size_t i = 0; i < op->getInputs().size(); ++i) {
                ptrs += (i ? ", " : "") + in(i);
                sizes.push_back(op->getInputs()[i]->getDims()[cc->getDim()]);
            }
            e.line("    const float *cins" + id + "[] = " + ptrs + "}; static const int cdims" + id +
                   "[] = " + e.ints(op->getOutputs()[0]->getDims()) + ", csz" + id +
                   "[] = " + e.ints(sizes) + ";");
            c << "pet_hip_concat(cins" << id << ", " << sizes.size() << ", " << out(0) << ", cdims"
              << id << ", " << op->getOutputs()[0]->getDims().size() << ", " << cc->getDim()
              << ", csz" << id << ", s)";
        } else if (auto pd = dynamic_cast<PadOp *>(op)) {
            std::string id = std::to_string(op->getGuid());
            e.line("    static const int pdims" + id + "[] = " +
                   e.ints(op->getInputs()[0]->getDims()) + ", pb" + id + "[] = " +
                   e.ints(pd->getBegin()) + ", pe" + id + "[] = " + e.ints(pd->getEnd()) + ";");
            c << "pet_hip_pad(" << in(0) << ", " << out(0) << ", pdims" << id << ", pb" << id
              << ", pe" << id << ", " << pd->getBegin().size() << ", s)";
        } else if (auto sl = dynamic_cast<SliceOp *>(op)) {
            std::string id = std::to_string(op->getGuid());
            e.line("    static const int ldims" + id + "[] = " +
                   e.ints(op->getInputs()[0]->getDims()) + ", lb" + id + "[] = " +
                   e.ints(sl->getBegin()) + ", le" + id + "[] = " + e.ints(sl->getEnd()) + ";");
            c << "pet_hip_slice(" << in(0) << ", " << out(0) << ", ldims" << id << ", lb" << id
              << ", le" << id << ", " << sl->getBegin().size() << ", s)";
        } else if (auto ex = dynamic_cast<ExtendOp *>(op)) {
            std::string id = std::to_string(op->getGuid());
            e.line("    static const int edims" + id + "[] = " +
                   e.ints(op->getInputs()[0]->getDims()) + ";");
            c << "pet_hip_extend(" << in(0) << ", " << out(0) << ", edims" << id << ", "
              << op->getInputs()[0]->getDims().size() << ", " << ex->getDim() << ", "
              << ex->getNum() << ", s)";
        } else if (dynamic_cast<EltwiseOp *>(op)) {
            std::string id = std::to_string(op->getGuid());
            std::string ptrs = "{", sizes = "{";
            for (size_t i = 0; i < op->getInputs().size(); ++i) {
                ptrs += (i ? ", " : "") + in(i);
                sizes += (i ? ", " : "") + std::to_string(op->getInputs()[i]->size());
            }
            e.line("    const float *eins" + id + "[] = " + ptrs + "}; static const size_t esz" + id +
                   "[] = " + sizes + "};");
            int code = op->getType() == Operator::Add   ? PET_HIP_ADD
                       : op->getType() == Operator::Sub ? PET_HIP_SUB
                       : op->getType() == Operator::Div ? PET_HIP_DIV
                                                        : PET_HIP_MUL;
            c << "pet_hip_eltwise(" << code << ", eins" << id << ", esz" << id << ", "
              << op->getInputs().size() << ", " << out(0) << ", " << op->getOutputs()[0]->size()
              << ", s)";
        } else if (auto ga = dynamic_cast<GatherOp *>(op)) {
            const Dim &d = op->getInputs()[0]->getDims();
            size_t pre = 1, post = 1;
            for (int i = 0; i < ga->getAxis(); ++i)
                pre *= (size_t)d[i];
            for (size_t i = ga->getAxis() + 1; i < d.size(); ++i)
                post *= (size_t)d[i];
            c << "pet_hip_gather(" << in(0) << ", " << in(1) << ", 1, " << out(0) << ", " << pre
              << ", " << d[ga->getAxis()] << ", " << post << ", " << op->getInputs()[1]->size()
              << ", s)";
        } else if (auto rm = dynamic_cast<ReduceMeanOp *>(op)) {
            const Dim &d = op->getInputs()[0]->getDims();
            size_t outer = 1, inner = 1;
            for (int i = 0; i < rm->getAxis(); ++i)
                outer *= (size_t)d[i];
            for (size_t i = rm->getAxis() + 1; i < d.size(); ++i)
                inner *= (size_t)d[i];
            c << "pet_hip_reduce_mean(" << in(0) << ", " << out(0) << ", " << outer << ", "
              << d[rm->getAxis()] << ", " << inner << ", s)";
        } else if (auto pw = dynamic_cast<PowOp *>(op)) {
            c << "pet_hip_pow(" << in(0) << ", " << out(0) << ", " << op->getInputs()[0]->size()
              << ", " << pw->getPow() << ", s)";
        } else if (auto bn = dynamic_cast<BatchNormOp *>(op)) {
            const Dim &d = op->getInputs()[0]->getDims();
            size_t inner = 1;
            for (size_t i = 2; i < d.size(); ++i)
                inner *= (size_t)d[i];
            char eps[32];
            snprintf(eps, sizeof eps, "%.9gf", bn->getEpsilon());
            c << "pet_hip_batchnorm(" << in(0) << ", " << e.name(bn->getScale()) << ", "
              << e.name(bn->getBias()) << ", " << e.name(bn->getMean()) << ", "
              << e.name(bn->getVar()) << ", " << out(0) << ", " << d[0] << ", " << d[1] << ", "
              << inner << ", " << eps << ", s)";
        } else if (auto act = dynamic_cast<ActivationOp *>(op)) {
            c << "pet_hip_activation(" << in(0) << ", " << out(0) << ", "
              << op->getInputs()[0]->size() << ", " << (int)act->getActType() << ", s)";
        } else if (auto pool = dynamic_cast<PoolOp *>(op)) {
            int kh, kw, ph, pw, sh, sw, dh, dw;
            std::tie(kh, kw, ph, pw, sh, sw, dh, dw) = pool->getArgs();
            auto d = op->getInputs()[0]->getDims();
            const unsigned fl = flagsOf(op);
            c << (fl ? "pet_hip_pool2d_ex(" : "pet_hip_pool2d(") << in(0) << ", " << out(0) << ", "
              << d[0] << ", " << d[1] << ", " << d[2] << ", " << d[3] << ", " << kh << ", " << kw
              << ", " << ph << ", " << pw << ", " << sh << ", " << sw << ", " << dh << ", " << dw
              << ", " << (op->getType() == Operator::MaxPool ? 0 : 1)
              << (fl ? ", " + std::to_string(fl) + "u" : std::string()) << ", s)";
        } else if (dynamic_cast<SoftmaxOp *>(op)) {
            size_t cols = (size_t)op->getInputs()[0]->getDims().back();
            c << "pet_hip_softmax(" << in(0) << ", " << out(0) << ", "
              << op->getInputs()[0]->size() / cols << ", " << cols << ", s)";
        } else if (dynamic_cast<ReshapeOp *>(op)) {
            c << "pet_hip_memcpy_d2d(" << out(0) << ", " << in(0) << ", "
              << op->getInputs()[0]->size() << " * sizeof(float), s)";
        } else {
            std::vector<std::string> setup;
            std::string call =
                op->emitLaunch([&](const Tensor *t) { return e.name(t); }, setup);
            if (call.empty())
                return false;
            c << call; // its set-up lines were written before the first launch
        }
        e.line("    CHECK(" + c.str() + "); // " + op->toString());
        return true;
    };

    e.line("    int odims[PET_HIP_MAX_RANK], orank = 0; (void)odims; (void)orank;");
    for (auto op : order) { // what such operators need before their first launch
        std::vector<std::string> setup;
        op->emitLaunch([&](const Tensor *t) { return e.name(t); }, setup);
        for (auto &l : setup)
            e.line("    " + l);
    }
    e.line("    // operators that only touch weights run once");
    for (auto op : order)
        if (weightOnly(op) && !skipped.count(op) && !rows.folded.count(op) &&
            !tails.absorbed.count(op) && !emitOp(op))
            return "";
    e.line("    // constant 3-D filters: kt-major copy where the backend has that form");
    for (auto op : order) {
        auto c3 = dynamic_cast<Conv3dOp *>(op);
        if (!c3 || skipped.count(op) || op->getInputs()[1]->getType() != Tensor::Weight)
            continue;
        Tensor *w = op->getInputs()[1];
        const Dim &wd = w->getDims();
        std::string n = e.name(w) + "_kt" + std::to_string(packedName.size());
        packedName[op] = n;
        std::ostringstream l;
        l << "    float *" << n << "; CHECK(pet_hip_malloc((void **)&" << n << ", " << w->size()
          << " * sizeof(float))); int " << n << "_ok = pet_hip_conv3d_pack_filters(" << e.name(w)
          << ", " << n << ", " << wd[0] << ", " << wd[1] << ", " << wd[2] << ", " << wd[3] << ", "
          << wd[4] << ", s) == PET_HIP_OK;";
        e.line(l.str());
    }
    e.line("    CHECK(pet_hip_stream_sync(s));");
    e.line("    // the rest is captured once and replayed as a HIP graph");
    e.line("    CHECK(pet_hip_graph_begin_capture(s));");
    if (!lp.fills.empty()) {
        e.line("    // outputs that accumulating contractions add into: their bias, in one launch");
        std::string l = "    const pet_hip_fill fills[] = {";
        for (size_t i = 0; i < lp.fills.size(); ++i) {
            const FillSpec &f = lp.fills[i];
            l += std::string(i ? ", " : "") + "{" + e.name(f.out) + ", " + nullable(e, f.bias) + ", " +
                 std::to_string(f.outer) + ", " + std::to_string(f.ch) + ", " +
                 std::to_string(f.inner) + "}";
        }
        e.line(l + "};");
        e.line("    CHECK(pet_hip_bias_fill_batch(fills, " + std::to_string(lp.fills.size()) +
               ", s));");
    }
    for (auto op : order)
        if (!weightOnly(op) && !skipped.count(op) && !rows.folded.count(op) &&
            !tails.absorbed.count(op) && !att.absorbed.count(op) && !views.folded.count(op) &&
            !emitOp(op))
            return "";
    e.line("    pet_hip_graph_t g; CHECK(pet_hip_graph_end_capture(s, &g));");
    e.line("    pet_hip_event_t st, ed; CHECK(pet_hip_event_create(&st)); "
           "CHECK(pet_hip_event_create(&ed));");
    e.line("    int warmup = 100, rounds = 1000;");
    e.line("    for (int i = 0; i < warmup + rounds; i++) {");
    e.line("        if (i == warmup) CHECK(pet_hip_event_record(st, s));");
    e.line("        CHECK(pet_hip_graph_launch(g, s));");
    e.line("    }");
    e.line("    CHECK(pet_hip_event_record(ed, s));");
    e.line("    CHECK(pet_hip_event_sync(ed));");
    e.line("    float duration; CHECK(pet_hip_event_elapsed_ms(&duration, st, ed));");
    e.line("    std::printf(\" Time(ms) : %f\\n\", duration / rounds);");
    e.line("    return 0;");
    e.line("}");
    return e.os.str();
}

int CodeEngine::genCode(std::shared_ptr<SubGraph> &graph, const std::string &filename) {
    std::string code = genCode(graph);
    if (code.empty())
        return 1;
    std::ofstream f(filename);
    if (!f)
        return 1;
    f << code;
    return 0;
}

} // namespace tpm
