#include "transpose.h"

#include <cstdio>
#include <sstream>

#include "pet_hip.h"

namespace tpm {

// Dim rules of the three micro-ops (the reference's putTranspose methods,
// src/Transpose/transpose.cc:22-42, 70-106, 136-150). The index algebra itself
// is evaluated by pet_hip_trans_chain on the device.
bool TransSplit::apply(std::vector<int> &dims, std::vector<int> &ops, std::vector<int> &) const {
    if (index < 0 || index >= (int)dims.size() || in_dim <= 0 || (extr && copys))
        return false;
    int outer;
    int inner;
    if (copys == 0) {
        outer = (dims[index] - 1) / (in_dim + extr) + 1;
        inner = in_dim;
    } else {
        if (dims[index] != 2 * in_dim)
            return false;
        outer = dims[index] / in_dim;
        inner = in_dim + copys;
    }
    dims[index] = outer;
    dims.insert(dims.begin() + index + 1, inner);
    ops.insert(ops.end(), {0, index, in_dim, extr, copys, 0});
    return true;
}

void TransSplit::print() const {
    std::printf("TransSplit(index=%d, in_dim=%d, extr=%d, copys=%d)\n", index, in_dim, extr, copys);
}

bool TransFuse::apply(std::vector<int> &dims, std::vector<int> &ops, std::vector<int> &) const {
    if (index < 0 || index + 1 >= (int)dims.size())
        return false;
    int in_dim = dims[index + 1];
    if (dels > 0) {
        if (pad != 0 || dims[index] != 2 || in_dim - dels <= 0)
            return false;
        dims[index] = dims[index] * (in_dim - dels);
    } else {
        dims[index] = dims[index] * (in_dim + pad) - pad;
    }
    dims.erase(dims.begin() + index + 1);
    ops.insert(ops.end(), {2, index, pad, dels, 0, 0});
    return true;
}

void TransFuse::print() const {
    std::printf("TransFuse(index=%d, pad=%d, dels=%d)\n", index, pad, dels);
}

bool TransReorder::apply(std::vector<int> &dims, std::vector<int> &ops,
                         std::vector<int> &perms) const {
    if (permu.size() != dims.size())
        return false;
    std::vector<int> nd(dims.size());
    std::vector<bool> seen(dims.size(), false);
    for (size_t i = 0; i < permu.size(); ++i) {
        int v = permu[i];
        if (v < 0 || v >= (int)dims.size() || seen[v])
            return false;
        seen[v] = true;
        nd[i] = dims[v];
    }
    dims = nd;
    ops.insert(ops.end(), {1, 0, 0, 0, 0, 0});
    perms.insert(perms.end(), permu.begin(), permu.end());
    return true;
}

void TransReorder::print() const {
    std::printf("TransReorder(");
    for (size_t i = 0; i < permu.size(); ++i)
        std::printf("%s%d", i ? "," : "", permu[i]);
    std::printf(")\n");
}

bool TransposeEngine::lower(const std::vector<std::shared_ptr<TransBasic>> &oper,
                            const std::vector<int> &inDims, TransProgram &out) const {
    out = TransProgram();
    out.inDims = inDims;
    std::vector<int> dims = inDims;
    for (auto &op : oper) {
        if (!op->apply(dims, out.ops, out.perms))
            return false;
        if (dims.size() > (size_t)PET_HIP_MAX_RANK)
            return false;
        out.nops++;
    }
    out.outDims = dims;
    return true;
}

std::string TransposeEngine::describe(const TransProgram &prog) const {
    std::ostringstream os;
    os << "in" << "[";
    for (size_t i = 0; i < prog.inDims.size(); ++i)
        os << (i ? "," : "") << prog.inDims[i];
    os << "] ->";
    size_t pp = 0;
    int rank = (int)prog.inDims.size();
    for (int o = 0; o < prog.nops; ++o) {
        const int *op = &prog.ops[6 * o];
        if (op[0] == 0) {
            os << " split(" << op[1] << "," << op[2] << ",extr=" << op[3] << ",copys=" << op[4]
               << ")";
            rank++;
        } else if (op[0] == 1) {
            os << " reorder(";
            for (int i = 0; i < rank; ++i)
                os << (i ? "," : "") << prog.perms[pp + i];
            os << ")";
            pp += rank;
        } else {
            os << " fuse(" << op[1] << ",pad=" << op[2] << ",dels=" << op[3] << ")";
            rank--;
        }
    }
    os << " -> out[";
    for (size_t i = 0; i < prog.outDims.size(); ++i)
        os << (i ? "," : "") << prog.outDims[i];
    os << "]";
    return os.str();
}

} // namespace tpm
