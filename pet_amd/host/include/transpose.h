// Micro-op lowering of TransposeOp chains (role of the reference's
// include/transpose.h). The reference composes a TVM lambda string from
// TransSplit / TransReorder / TransFuse; here the same three micro-ops, with
// the same boundary-correction parameters, are encoded for
// pet_hip_trans_chain, which evaluates the index algebra on the device.
#pragma once
#include <memory>
#include <string>
#include <vector>

namespace tpm {

class TransBasic {
  public:
    virtual ~TransBasic() {}
    // Applies the micro-op to `dims` and appends its encoding: six ints to
    // `ops`, and for a reorder its permutation to `perms`.
    virtual bool apply(std::vector<int> &dims, std::vector<int> &ops,
                       std::vector<int> &perms) const = 0;
    virtual void print() const = 0;
};

// (..., d, ...) -> (..., d / in_dim, in_dim, ...); extr: stride in_dim + extr
// between blocks; copys: each half carries `copys` halo rows.
class TransSplit : public TransBasic {
    int index, in_dim, extr, copys;

  public:
    TransSplit(int index, int in_dim, int extr = 0, int copys = 0)
        : index(index), in_dim(in_dim), extr(extr), copys(copys) {}
    bool apply(std::vector<int> &dims, std::vector<int> &ops, std::vector<int> &perms) const override;
    void print() const override;
};

// (..., a, b, ...) -> (..., a * b, ...); pad: zero rows between blocks;
// dels: rows dropped at the seam.
class TransFuse : public TransBasic {
    int index, pad, dels;

  public:
    TransFuse(int index, int pad = 0, int dels = 0) : index(index), pad(pad), dels(dels) {}
    bool apply(std::vector<int> &dims, std::vector<int> &ops, std::vector<int> &perms) const override;
    void print() const override;
};

class TransReorder : public TransBasic {
    std::vector<int> permu;

  public:
    explicit TransReorder(std::vector<int> permu) : permu(std::move(permu)) {}
    bool apply(std::vector<int> &dims, std::vector<int> &ops, std::vector<int> &perms) const override;
    void print() const override;
};

// A lowered chain, ready for pet_hip_trans_chain.
struct TransProgram {
    std::vector<int> inDims, outDims;
    std::vector<int> ops;   // 6 ints per micro-op
    std::vector<int> perms; // permutations of the reorders, concatenated
    int nops = 0;
};

class TransposeEngine {
    TransposeEngine() {}

  public:
    static TransposeEngine &getInstance() {
        static TransposeEngine e;
        return e;
    }
    // Lowers a micro-op list on `inDims`; returns false for an ill-formed chain.
    bool lower(const std::vector<std::shared_ptr<TransBasic>> &oper, const std::vector<int> &inDims,
               TransProgram &out) const;
    // Human-readable index map "out[a,b,..] = in[..]" (what getLambda printed for TVM).
    std::string describe(const TransProgram &prog) const;
};

} // namespace tpm
