// MemBoundOp (role of the reference's include/operator.h:2009-2100): a memory-bound
// operator whose outputs are given by an expression of the reference's nnet tree. Only
// included where that tree's headers are on the include path (see operator.h); everything
// is inline, so the class lives in whatever is built against the tree, not in the host
// library.
//
// The reference evaluates the expression on the host with nnet::Interpreter
// (src/Graph/operator.cc:3601-3644) and prints a TVM kernel for the GPU
// (src/Graph/code_engine.cc:1752-1798). Here the tree is flattened once into the integer
// program of pet_hip.h and every compute / launch runs it on the device.
#pragma once
#include <cstring>
#include <map>

namespace tpm {

// Flattens an nnet expression into the stack-machine program of pet_hip.h.
class NnetLowering {
  public:
    // The program for `expr` (a RangeOp) reading `nnetInputs` (tensor t of the program is
    // nnetInputs[t]); empty on expressions the program format cannot hold.
    static std::vector<int> lower(const nnet::Expr &expr,
                                  const std::vector<nnet::Tensor> &nnetInputs) {
        NnetLowering l;
        for (size_t i = 0; i < nnetInputs.size(); ++i)
            l.tensorOf[nnetInputs[i]->getName()] = (int)i;
        auto range = nnet::as<nnet::RangeOpNode>(expr);
        if (!range || nnetInputs.size() > 8)
            return {};
        l.code = {(int)PET_HIP_EXPR_MAGIC, (int)nnetInputs.size()};
        for (auto &t : nnetInputs) {
            l.code.push_back(t->getDims());
            for (int d : t->getShape())
                l.code.push_back(d);
        }
        // one output position per loop iterator; MemBoundOp::compute counts them from 0
        const auto &loops = range->getLoopVarRanges();
        l.code.push_back((int)loops.size());
        for (auto &vr : loops)
            l.code.push_back(vr.second.second - vr.second.first);
        if (!l.emitRange(range, /*top=*/true))
            return {};
        l.code.push_back(PET_HIP_EXPR_END);
        return l.code;
    }

  private:
    typedef std::map<std::string, int> Scope;
    std::vector<int> code;
    std::map<std::string, int> tensorOf;
    int slots = 0;

    static bool isIndex(const nnet::Expr &e) {
        switch (e->getType()) {
        case nnet::NodeType::ConstantNodeType:
        case nnet::NodeType::VarNodeType:
            return true;
        case nnet::NodeType::BinaryOpNodeType: {
            auto b = nnet::as<nnet::BinaryOpNode>(e);
            return isIndex(b->getLhs()) && isIndex(b->getRhs());
        }
        default:
            return false;
        }
    }

    bool emitIndex(const nnet::Expr &e, const Scope &scope) {
        if (auto c = nnet::as<nnet::ConstantNode>(e)) {
            code.push_back(PET_HIP_EXPR_ICONST);
            code.push_back(c->getValue());
            return true;
        }
        if (auto v = nnet::as<nnet::VarNode>(e)) {
            auto it = scope.find(v->getName());
            if (it == scope.end())
                return false;
            code.push_back(PET_HIP_EXPR_IVAR);
            code.push_back(it->second);
            return true;
        }
        auto b = nnet::as<nnet::BinaryOpNode>(e);
        if (!b || !emitIndex(b->getLhs(), scope) || !emitIndex(b->getRhs(), scope))
            return false;
        switch (b->getOpType()) {
        case nnet::OpType::Add:
            code.push_back(PET_HIP_EXPR_IADD);
            break;
        case nnet::OpType::Sub:
            code.push_back(PET_HIP_EXPR_ISUB);
            break;
        case nnet::OpType::Mul:
            code.push_back(PET_HIP_EXPR_IMUL);
            break;
        case nnet::OpType::Div:
            code.push_back(PET_HIP_EXPR_IDIV);
            break;
        case nnet::OpType::Mod:
            code.push_back(PET_HIP_EXPR_IMOD);
            break;
        default:
            return false;
        }
        return true;
    }

    bool emitSubscript(const nnet::Subscript &s, const Scope &scope) {
        for (auto &idx : s->getIndex())
            if (!isIndex(idx) || !emitIndex(idx, scope))
                return false;
        nnet::Expr obj = s->getObject();
        if (auto r = nnet::as<nnet::RangeOpNode>(obj))
            return emitRange(r, false);
        auto t = nnet::as<nnet::TensorNode>(obj);
        if (!t || !tensorOf.count(t->getName()) ||
            (size_t)t->getDims() != s->getIndex().size())
            return false;
        code.push_back(PET_HIP_EXPR_LOAD);
        code.push_back(tensorOf[t->getName()]);
        return true;
    }

    bool emitValue(const nnet::Expr &e, const Scope &scope) {
        if (isIndex(e)) {
            if (!emitIndex(e, scope))
                return false;
            code.push_back(PET_HIP_EXPR_I2F);
            return true;
        }
        if (auto s = nnet::as<nnet::SubscriptNode>(e))
            return emitSubscript(s, scope);
        if (auto f = nnet::as<nnet::FuncNode>(e)) {
            if (!emitSubscript(f->getObject(), scope))
                return false;
            code.push_back(f->getFuncType() == nnet::FuncType::Relu ? PET_HIP_EXPR_FRELU
                                                                    : PET_HIP_EXPR_FTANH);
            return true;
        }
        if (auto b = nnet::as<nnet::BinaryOpNode>(e)) {
            if (!emitValue(b->getLhs(), scope) || !emitValue(b->getRhs(), scope))
                return false;
            switch (b->getOpType()) {
            case nnet::OpType::Add:
                code.push_back(PET_HIP_EXPR_FADD);
                break;
            case nnet::OpType::Sub:
                code.push_back(PET_HIP_EXPR_FSUB);
                break;
            case nnet::OpType::Mul:
                code.push_back(PET_HIP_EXPR_FMUL);
                break;
            case nnet::OpType::Div:
                code.push_back(PET_HIP_EXPR_FDIV);
                break;
            case nnet::OpType::Mod:
                code.push_back(PET_HIP_EXPR_FMOD);
                break;
            default:
                return false;
            }
            return true;
        }
        return false; // a bare RangeOp or Tensor is not a value
    }

    // Positions of the loop iterators are on the integer stack. For the top range they
    // count from 0 whatever the iterators' own ranges (MemBoundOp::compute,
    // src/Graph/operator.cc:3625-3633, hands the interpreter 0-based positions, which its
    // range checks then require to lie in [left, right): only ranges that start at 0 pass).
    bool emitRange(const nnet::RangeOp &r, bool top) {
        Scope scope;
        const auto &loops = r->getLoopVarRanges();
        const auto &sums = r->getSumVarRanges();
        if (loops.size() > PET_HIP_MAX_RANK || sums.size() > PET_HIP_MAX_RANK)
            return false;
        for (auto &vr : loops)
            scope[vr.first->getName()] = slots++;
        for (auto &vr : sums)
            scope[vr.first->getName()] = slots++;
        if (slots > 32)
            return false;
        if (top)
            for (auto &vr : loops)
                if (vr.second.first != 0)
                    return false;
        const size_t at = code.size();
        code.push_back(PET_HIP_EXPR_RANGE);
        code.push_back((int)loops.size());
        code.push_back(-1);
        const std::vector<int> pads = r->getPaddings();
        for (size_t i = 0; i < loops.size(); ++i) {
            code.push_back(scope[loops[i].first->getName()]);
            code.push_back(loops[i].second.first);
            code.push_back(loops[i].second.second);
            code.push_back(i < pads.size() ? pads[i] : 0);
        }
        if (!sums.empty()) {
            code.push_back(PET_HIP_EXPR_SUM);
            code.push_back((int)sums.size());
            for (auto &vr : sums) {
                if (vr.second.first >= vr.second.second)
                    return false;
                code.push_back(scope[vr.first->getName()]);
                code.push_back(vr.second.first);
                code.push_back(vr.second.second);
            }
            const int body = (int)code.size();
            if (!emitValue(r->getSummand(), scope))
                return false;
            code.push_back(PET_HIP_EXPR_SUMEND);
            code.push_back((int)sums.size());
            code.push_back(body);
            for (auto &vr : sums) {
                code.push_back(scope[vr.first->getName()]);
                code.push_back(vr.second.first);
                code.push_back(vr.second.second);
            }
        } else if (!emitValue(r->getSummand(), scope)) {
            return false;
        }
        code[at + 2] = (int)code.size();
        return true;
    }
};

class MemBoundOp : public Operator {
  public:
    MemBoundOp(const TensorVec &input, const TensorVec &output,
               const std::vector<nnet::Tensor> &nnetInputs, nnet::Expr expr, double exec_time,
               std::string hint = {})
        : Operator(MemBound, input, output), nnetInputs(nnetInputs), expr(expr),
          exec_time(exec_time), hint(hint) {
        initHash();
        assert(!outputs.empty());
        setWeight();
    }
    MemBoundOp(const MemBoundOp &rhs)
        : Operator(rhs), nnetInputs(rhs.nnetInputs), expr(rhs.expr), exec_time(rhs.exec_time),
          hint(rhs.hint), n(rhs.n), f(rhs.f), h(rhs.h), w(rhs.w) {}
    ~MemBoundOp() override {
        if (deviceCode)
            pet_hip_free(deviceCode);
    }
    MemBoundOp *clone() override { return new MemBoundOp(*this); }

    Dim computeShape() override { return outputs[0]->getDims(); }

    // The reference returns the estimate its derivation attached (include/operator.h:
    // 2051-2053); here the operator is launched and timed like every other one, so that the
    // search ranks by measured cost. Operators that only touch weights cost nothing, as
    // upstream: they run once, ahead of inference.
    double perf(PerfEngine *pe, int rounds = 200, int warmupRounds = 200) override {
        if (isComputeWeight())
            return 0;
        if (!expr) {
            // A placeholder the reference's transforms leave for a layout move they only
            // price (src/nnet/nmutator.cc:529-567: no expression, a time from the bytes moved
            // at 200 GiB/s): the same bytes at this GPU's measured copy bandwidth.
            const double bw = pe ? pe->layoutBandwidthGiBs() : 0.0;
            return bw > 0 ? exec_time * 200.0 / bw : exec_time;
        }
        if (measured < 0) {
            for (auto t : outputs)
                if (t->devicePtr() == nullptr)
                    return INFINITY;
            measured = timeLaunches(std::min(rounds, 50), std::min(warmupRounds, 10));
        }
        return measured;
    }
    double getEstimatedTime() const { return exec_time; }

    int launch(pet_hip_stream_t stream) override {
        if (!ensureProgram())
            return PET_HIP_ERR_UNSUPPORTED;
        if (inputs.size() != nnetInputs.size() || inputs.size() > 8)
            return PET_HIP_ERR_INVALID;
        const float *ins[8];
        for (size_t i = 0; i < inputs.size(); ++i)
            ins[i] = inputs[i]->devicePtr();
        return pet_hip_expr_f32(code.data(), (int)code.size(), deviceCode, ins,
                                (int)inputs.size(), outputs[0]->devicePtr(), stream);
    }

    std::string emitLaunch(const std::function<std::string(const Tensor *)> &name,
                           std::vector<std::string> &setup) const override {
        std::vector<int> prog = NnetLowering::lower(expr, nnetInputs);
        if (prog.empty())
            return "";
        const std::string id = std::to_string(getGuid());
        std::string words = "{";
        for (size_t i = 0; i < prog.size(); ++i)
            words += (i ? ", " : "") + std::to_string(prog[i]);
        std::string ptrs = "{";
        for (size_t i = 0; i < inputs.size(); ++i)
            ptrs += (i ? ", " : "") + name(inputs[i]);
        setup.push_back("static const int mb" + id + "[] = " + words + "}; int *mbdev" + id +
                        "; CHECK(pet_hip_expr_program_create(mb" + id + ", " +
                        std::to_string(prog.size()) + ", &mbdev" + id + "));");
        setup.push_back("const float *mbin" + id + "[] = " + ptrs + "};");
        return "pet_hip_expr_f32(mb" + id + ", " + std::to_string(prog.size()) + ", mbdev" + id +
               ", mbin" + id + ", " + std::to_string(inputs.size()) + ", " + name(outputs[0]) +
               ", s)";
    }

    std::string toString() const override {
        std::ostringstream os;
        os << "MemBound[" << hash << "](";
        for (size_t i = 0; i < inputs.size(); ++i)
            os << "i" << i << "=" << inputs[i]->getHash() << (i + 1 < inputs.size() ? " " : "");
        os << ", ";
        for (size_t i = 0; i < outputs.size(); ++i)
            os << "o" << i << "=" << outputs[i]->getHash() << (i + 1 < outputs.size() ? " " : "");
        os << ", exec_time=" << exec_time << ", NNet Inputs=[";
        for (const auto &tensor : nnetInputs)
            os << tensor->toReadable() << ",";
        os << "])";
        return os.str();
    }
    int numInputs() override { return (int)inputs.size(); }
    int numOutputs() override { return (int)outputs.size(); }

    const std::vector<nnet::Tensor> &getNnetInputs() const { return nnetInputs; }
    nnet::Expr getExpr() const { return expr; }
    bool isComputeWeight() const {
        for (auto input : inputs)
            if (input->getType() != Tensor::Weight)
                return false;
        return true;
    }
    const std::string &getHint() const { return hint; }
    void setNFHW(int _n, int _f, int _h, int _w) { n = _n, f = _f, h = _h, w = _w; }
    std::tuple<int, int, int, int> getNFHW() const { return {n, f, h, w}; }
    // The flattened program (empty when the expression does not fit the format).
    const std::vector<int> &program() {
        ensureProgram();
        return code;
    }

  private:
    bool checkValid(const TensorVec &) override { return true; }
    void initHash() override {
        hash = type;
        uint64_t bits = 0;
        static_assert(sizeof(bits) == sizeof(exec_time), "double is 64 bits");
        std::memcpy(&bits, &exec_time, sizeof(bits));
        hash = hashAppend(hash, bits);
        hash = hashPack(hash);
    }
    void setWeight() {
        if (isComputeWeight())
            for (auto output : outputs)
                output->setType(Tensor::Weight);
    }
    bool ensureProgram() {
        if (deviceCode)
            return true;
        if (code.empty())
            code = NnetLowering::lower(expr, nnetInputs);
        if (code.empty() || !petInit())
            return false;
        return pet_hip_expr_program_create(code.data(), (int)code.size(), &deviceCode) ==
               PET_HIP_OK;
    }

    std::vector<nnet::Tensor> nnetInputs;
    nnet::Expr expr;
    double exec_time;
    std::string hint;
    int n = 0, f = 0, h = 0, w = 0;
    std::vector<int> code;     // the flattened expression
    int *deviceCode = nullptr; // its device copy, owned
    double measured = -1;
};

} // namespace tpm
