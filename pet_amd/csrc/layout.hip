// Layout operators of the C ABI: each one is lowered on the host into a
// ViewDesc and handed to the view-copy engine; transpose chains that do not
// fit one div/mod level per dim run through an on-device interpreter instead.
#include "view.h"

#include <algorithm>
#include <vector>

using namespace pet;

namespace {

long long prod(const int *d, int n) {
    long long p = 1;
    for (int i = 0; i < n; ++i)
        p *= d[i];
    return p;
}

bool dims_ok(const int *d, int rank) {
    if (!d || rank < 1 || rank > PET_HIP_MAX_RANK)
        return false;
    for (int i = 0; i < rank; ++i)
        if (d[i] < 0)
            return false;
    return true;
}

ViewDim plain_dim(int ext, long long os, long long sr) {
    ViewDim d;
    d.ext = ext;
    d.m = ext > 0 ? ext : 1;
    d.lo = 0;
    d.hi = ext;
    d.os = os;
    d.sq = 0;
    d.sr = sr;
    return d;
}

// ---- transpose chain ---------------------------------------------------------

constexpr int kMaxChainOps = 15;

struct ChainOp {
    int kind, a, b, c, d;
    int perm[PET_HIP_MAX_RANK];
    int in_dim; // fuse: extent of dim index+1 before the fuse
};

struct ChainProgram {
    int nops, in_rank, out_rank;
    ChainOp op[kMaxChainOps];
    int dims[kMaxChainOps + 1][PET_HIP_MAX_RANK];
    int ranks[kMaxChainOps + 1];
};

// Forward pass over the dims, the rules of TransSplit / TransReorder /
// TransFuse::putTranspose.
int build_chain(const int *in_dims, int rank, const int *ops, int nops, const int *perms,
                ChainProgram &cp) {
    if (nops < 0 || nops > kMaxChainOps)
        return set_error(PET_HIP_ERR_INVALID, "transpose chain has %d ops (max %d)", nops,
                         kMaxChainOps);
    if (!dims_ok(in_dims, rank))
        return set_error(PET_HIP_ERR_INVALID, "bad input dims");
    cp.nops = nops;
    cp.in_rank = rank;
    for (int i = 0; i < rank; ++i)
        cp.dims[0][i] = in_dims[i];
    cp.ranks[0] = rank;
    const int *pp = perms;
    for (int o = 0; o < nops; ++o) {
        const int *src = ops + 6 * o;
        ChainOp &op = cp.op[o];
        op.kind = src[0];
        op.a = src[1];
        op.b = src[2];
        op.c = src[3];
        op.d = src[4];
        op.in_dim = 0;
        const int *s = cp.dims[o];
        int *d = cp.dims[o + 1];
        int rk = cp.ranks[o];
        if (op.kind == 0) {
            int index = op.a, in_dim = op.b, extr = op.c, copys = op.d;
            if (rk >= PET_HIP_MAX_RANK || index < 0 || index >= rk || in_dim <= 0 || extr < 0 ||
                copys < 0 || (extr != 0 && copys != 0))
                return set_error(PET_HIP_ERR_INVALID, "bad split micro-op %d", o);
            for (int i = 0; i <= index; ++i)
                d[i] = s[i];
            for (int i = index + 1; i < rk; ++i)
                d[i + 1] = s[i];
            if (copys == 0) {
                d[index + 1] = in_dim;
                d[index] = (s[index] - 1) / (in_dim + extr) + 1;
            } else {
                if (s[index] != in_dim * 2)
                    return set_error(PET_HIP_ERR_INVALID,
                                     "halo split needs dim == 2 * in_dim (micro-op %d)", o);
                d[index + 1] = in_dim + copys;
                d[index] = s[index] / in_dim;
            }
            cp.ranks[o + 1] = rk + 1;
        } else if (op.kind == 1) {
            if (!pp)
                return set_error(PET_HIP_ERR_INVALID, "reorder without a permutation");
            bool seen[PET_HIP_MAX_RANK] = {false};
            for (int i = 0; i < rk; ++i) {
                int v = pp[i];
                if (v < 0 || v >= rk || seen[v])
                    return set_error(PET_HIP_ERR_INVALID, "bad permutation in micro-op %d", o);
                seen[v] = true;
                op.perm[i] = v;
                d[i] = s[v];
            }
            pp += rk;
            cp.ranks[o + 1] = rk;
        } else if (op.kind == 2) {
            int index = op.a, pad = op.b, dels = op.c;
            if (index < 0 || index + 1 >= rk || pad < 0 || dels < 0)
                return set_error(PET_HIP_ERR_INVALID, "bad fuse micro-op %d", o);
            int in_dim = s[index + 1];
            op.in_dim = in_dim;
            for (int i = 0; i < index; ++i)
                d[i] = s[i];
            if (dels > 0) {
                if (pad != 0 || s[index] != 2 || in_dim - dels <= 0)
                    return set_error(PET_HIP_ERR_INVALID,
                                     "drop fuse needs pad == 0 and an outer dim of 2 (micro-op %d)",
                                     o);
                d[index] = s[index] * (in_dim - dels);
            } else {
                d[index] = s[index] * (in_dim + pad) - pad;
            }
            for (int i = index + 2; i < rk; ++i)
                d[i - 1] = s[i];
            cp.ranks[o + 1] = rk - 1;
        } else {
            return set_error(PET_HIP_ERR_INVALID, "unknown micro-op kind %d", op.kind);
        }
    }
    cp.out_rank = cp.ranks[nops];
    return PET_HIP_OK;
}

// A dim of an intermediate stage as an affine form over "primitive" variables:
// every output dim contributes its q part and its r part.
struct Affine {
    long long cq[PET_HIP_MAX_RANK]; // coefficient of q_j
    long long cr[PET_HIP_MAX_RANK]; // coefficient of r_j
    long long c0;
};

// Tries to express the chain as a ViewDesc over the output index space. Returns
// false when some dim would need more than one div/mod level or when an index
// could leave its range (the interpreter handles those).
bool compile_chain(const ChainProgram &cp, ViewDesc &v) {
    const int R = cp.out_rank;
    const int *out = cp.dims[cp.nops];
    int m[PET_HIP_MAX_RANK], hi[PET_HIP_MAX_RANK];
    bool split_used[PET_HIP_MAX_RANK];
    Affine cur[PET_HIP_MAX_RANK], nxt[PET_HIP_MAX_RANK];
    for (int j = 0; j < R; ++j) {
        m[j] = out[j] > 0 ? out[j] : 1; // no div: q == 0, r == idx
        hi[j] = out[j];
        split_used[j] = false;
        memset(&cur[j], 0, sizeof(Affine));
        cur[j].cr[j] = 1;
    }
    auto range = [&](const Affine &a, long long &lo_, long long &hi_) {
        lo_ = hi_ = a.c0;
        for (int j = 0; j < R; ++j) {
            long long qmax = split_used[j] ? (out[j] - 1) / m[j] : 0;
            long long rmax = std::min(split_used[j] ? m[j] : out[j], hi[j]) - 1;
            if (rmax < 0)
                rmax = 0;
            long long e = a.cq[j] * qmax;
            (e < 0 ? lo_ : hi_) += e;
            e = a.cr[j] * rmax;
            (e < 0 ? lo_ : hi_) += e;
        }
    };
    int rk = R;
    for (int o = cp.nops - 1; o >= 0; --o) {
        const ChainOp &op = cp.op[o];
        const int *s = cp.dims[o];
        int prk = cp.ranks[o];
        if (op.kind == 0) {
            int index = op.a, in_dim = op.b, extr = op.c, copys = op.d;
            long long mul = copys == 0 ? (in_dim + extr) : (in_dim - copys);
            for (int i = 0; i < index; ++i)
                nxt[i] = cur[i];
            Affine e;
            for (int j = 0; j < R; ++j) {
                e.cq[j] = cur[index].cq[j] * mul + cur[index + 1].cq[j];
                e.cr[j] = cur[index].cr[j] * mul + cur[index + 1].cr[j];
            }
            e.c0 = cur[index].c0 * mul + cur[index + 1].c0;
            nxt[index] = e;
            for (int i = index + 1; i < prk; ++i)
                nxt[i] = cur[i + 1];
        } else if (op.kind == 1) {
            for (int i = 0; i < prk; ++i)
                nxt[op.perm[i]] = cur[i];
        } else {
            int index = op.a, pad = op.b, dels = op.c;
            int in_dim = op.in_dim;
            // the fused dim must be exactly one untouched output dim
            const Affine &e = cur[index];
            int var = -1;
            for (int j = 0; j < R; ++j) {
                if (e.cq[j] != 0)
                    return false;
                if (e.cr[j] != 0) {
                    if (var >= 0 || e.cr[j] != 1)
                        return false;
                    var = j;
                }
            }
            if (var < 0 || e.c0 != 0 || split_used[var])
                return false;
            split_used[var] = true;
            for (int i = 0; i < index; ++i)
                nxt[i] = cur[i];
            Affine q, r;
            memset(&q, 0, sizeof(q));
            memset(&r, 0, sizeof(r));
            q.cq[var] = 1;
            r.cr[var] = 1;
            if (dels > 0) {
                m[var] = in_dim - dels;
                r.cq[var] = dels; // r + q * dels
            } else {
                m[var] = in_dim + pad;
                hi[var] = std::min(hi[var], in_dim);
            }
            nxt[index] = q;
            nxt[index + 1] = r;
            for (int i = index + 2; i < prk; ++i)
                nxt[i] = cur[i - 1];
        }
        rk = prk;
        for (int i = 0; i < rk; ++i) {
            cur[i] = nxt[i];
            long long lo_, hi_;
            range(cur[i], lo_, hi_);
            if (lo_ < 0 || hi_ >= s[i])
                return false;
        }
    }
    long long istr[PET_HIP_MAX_RANK], ostr[PET_HIP_MAX_RANK];
    row_major_strides(cp.dims[0], cp.in_rank, istr);
    row_major_strides(out, R, ostr);
    v.rank = R;
    v.ibase = 0;
    v.obase = 0;
    for (int j = 0; j < R; ++j) {
        ViewDim &d = v.d[j];
        d.ext = out[j];
        d.m = split_used[j] ? m[j] : (out[j] > 0 ? out[j] : 1);
        d.lo = 0;
        d.hi = hi[j];
        d.os = ostr[j];
        d.sq = 0;
        d.sr = 0;
    }
    for (int i = 0; i < cp.in_rank; ++i) {
        v.ibase += cur[i].c0 * istr[i];
        for (int j = 0; j < R; ++j) {
            v.d[j].sq += cur[i].cq[j] * istr[i];
            v.d[j].sr += cur[i].cr[j] * istr[i];
        }
    }
    return true;
}

// A chain without correction parameters only regroups and reorders extents: each
// dim is a run of factors (extent, input stride), a split cuts a run, a reorder
// moves runs, a fuse joins two. The output is then a plain strided view whose
// dims are the factors in their final order, however many times a dim was fused.
bool compile_pure_chain(const ChainProgram &cp, ViewDesc &v) {
    struct Factor {
        long long ext, stride;
    };
    std::vector<std::vector<Factor>> dims(cp.in_rank);
    long long istr[PET_HIP_MAX_RANK];
    row_major_strides(cp.dims[0], cp.in_rank, istr);
    for (int i = 0; i < cp.in_rank; ++i) {
        if (cp.dims[0][i] <= 0)
            return false;
        dims[i].push_back({cp.dims[0][i], istr[i]});
    }
    for (int o = 0; o < cp.nops; ++o) {
        const ChainOp &op = cp.op[o];
        if (op.kind == 0) {
            if (op.c != 0 || op.d != 0 || cp.dims[o][op.a] % op.b != 0)
                return false;
            std::vector<Factor> &outer = dims[op.a], inner;
            long long need = op.b;
            while (need > 1) {
                if (outer.empty())
                    return false;
                Factor last = outer.back();
                if (last.ext <= need) {
                    if (need % last.ext != 0)
                        return false;
                    inner.insert(inner.begin(), last);
                    need /= last.ext;
                    outer.pop_back();
                } else {
                    if (last.ext % need != 0)
                        return false;
                    inner.insert(inner.begin(), {need, last.stride});
                    outer.back() = {last.ext / need, last.stride * need};
                    need = 1;
                }
            }
            dims.insert(dims.begin() + op.a + 1, inner);
        } else if (op.kind == 1) {
            std::vector<std::vector<Factor>> moved(dims.size());
            for (size_t i = 0; i < dims.size(); ++i)
                moved[i] = dims[op.perm[i]];
            dims.swap(moved);
        } else {
            if (op.b != 0 || op.c != 0)
                return false;
            std::vector<Factor> &head = dims[op.a], &tail = dims[op.a + 1];
            head.insert(head.end(), tail.begin(), tail.end());
            dims.erase(dims.begin() + op.a + 1);
        }
    }
    std::vector<Factor> flat;
    for (auto &run : dims)
        for (auto &f : run)
            if (f.ext != 1)
                flat.push_back(f);
    if (flat.empty())
        flat.push_back({1, 1});
    if (flat.size() > (size_t)PET_HIP_MAX_RANK)
        return false;
    v.rank = (int)flat.size();
    v.ibase = 0;
    v.obase = 0;
    long long os = 1;
    for (int j = v.rank - 1; j >= 0; --j) {
        if (flat[j].ext > 0x7fffffffll)
            return false;
        v.d[j] = plain_dim((int)flat[j].ext, os, flat[j].stride);
        os *= flat[j].ext;
    }
    return true;
}

// Fallback: undo the chain per output element on the device.
__global__ __launch_bounds__(256) void chain_interp_kernel(const float *__restrict__ x,
                                                           float *__restrict__ y,
                                                           ChainProgram cp, unsigned total) {
    unsigned oi = blockIdx.x * 256u + threadIdx.x;
    const unsigned step = gridDim.x * 256u;
    const int ork = cp.out_rank;
    for (; oi < total; oi += step) {
        int v[PET_HIP_MAX_RANK], u[PET_HIP_MAX_RANK];
        unsigned tmp = oi;
        for (int j = ork - 1; j >= 0; --j) {
            unsigned e = (unsigned)cp.dims[cp.nops][j];
            v[j] = (int)(tmp % e);
            tmp /= e;
        }
        bool ok = true;
        for (int o = cp.nops - 1; o >= 0 && ok; --o) {
            const ChainOp &op = cp.op[o];
            const int rk = cp.ranks[o];
            if (op.kind == 0) {
                int index = op.a;
                int a = v[index], b = v[index + 1];
                for (int i = 0; i < index; ++i)
                    u[i] = v[i];
                u[index] = op.d == 0 ? a * (op.b + op.c) + b : a * op.b + b - a * op.d;
                for (int i = index + 1; i < rk; ++i)
                    u[i] = v[i + 1];
            } else if (op.kind == 1) {
                for (int i = 0; i < rk; ++i)
                    u[op.perm[i]] = v[i];
            } else {
                int index = op.a, pad = op.b, dels = op.c, in_dim = op.in_dim;
                int a = v[index];
                for (int i = 0; i < index; ++i)
                    u[i] = v[i];
                if (dels > 0) {
                    u[index] = a / (in_dim - dels);
                    u[index + 1] = a % (in_dim - dels) + (a / (in_dim - dels)) * dels;
                } else {
                    u[index] = a / (in_dim + pad);
                    u[index + 1] = a % (in_dim + pad);
                    if (u[index + 1] >= in_dim)
                        ok = false;
                }
                for (int i = index + 2; i < rk; ++i)
                    u[i] = v[i - 1];
            }
            for (int i = 0; i < rk; ++i) {
                v[i] = u[i];
                if (v[i] < 0 || v[i] >= cp.dims[o][i])
                    ok = false;
            }
        }
        float val = 0.f;
        if (ok) {
            long long io = 0;
            for (int i = 0; i < cp.in_rank; ++i)
                io = io * cp.dims[0][i] + v[i];
            val = x[io];
        }
        y[oi] = val;
    }
}

} // namespace

extern "C" {

int pet_hip_transpose(const float *x, float *y, const int *flat_dims, const int *perm, int nflat,
                      pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (!dims_ok(flat_dims, nflat) || !perm)
        return set_error(PET_HIP_ERR_INVALID, "bad flat dims / perm");
    bool seen[PET_HIP_MAX_RANK] = {false};
    for (int i = 0; i < nflat; ++i) {
        if (perm[i] < 0 || perm[i] >= nflat || seen[perm[i]])
            return set_error(PET_HIP_ERR_INVALID, "perm is not a permutation");
        seen[perm[i]] = true;
    }
    long long istr[PET_HIP_MAX_RANK];
    row_major_strides(flat_dims, nflat, istr);
    ViewDesc v;
    v.rank = nflat;
    v.ibase = v.obase = 0;
    long long os = 1;
    for (int j = nflat - 1; j >= 0; --j) {
        v.d[j] = plain_dim(flat_dims[perm[j]], os, istr[perm[j]]);
        os *= flat_dims[perm[j]];
    }
    long long total = prod(flat_dims, nflat);
    return launch_view_copy(x, y, v, total, total, as_stream(stream));
}

int pet_hip_trans_chain(const float *x, float *y, const int *in_dims, int rank, const int *ops,
                        int nops, const int *perms, int *out_dims, int *out_rank,
                        pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (nops > 0 && !ops)
        return set_error(PET_HIP_ERR_INVALID, "null micro-op list");
    ChainProgram cp;
    memset(&cp, 0, sizeof(cp));
    int rc = build_chain(in_dims, rank, ops, nops, perms, cp);
    if (rc)
        return rc;
    if (out_rank)
        *out_rank = cp.out_rank;
    if (out_dims)
        for (int i = 0; i < cp.out_rank; ++i)
            out_dims[i] = cp.dims[nops][i];
    for (int i = 0; i < cp.out_rank; ++i)
        if (cp.dims[nops][i] < 0)
            return set_error(PET_HIP_ERR_INVALID, "chain produces a negative extent");
    if (!y)
        return PET_HIP_OK;
    long long in_total = prod(cp.dims[0], cp.in_rank);
    long long out_total = prod(cp.dims[nops], cp.out_rank);
    if (out_total == 0)
        return PET_HIP_OK;
    ViewDesc v;
    if (compile_pure_chain(cp, v) || compile_chain(cp, v))
        return launch_view_copy(x, y, v, in_total, out_total, as_stream(stream));
    if (!x)
        return set_error(PET_HIP_ERR_INVALID, "null tensor pointer");
    if (in_total >= (1ll << 31) || out_total >= (1ll << 31))
        return set_error(PET_HIP_ERR_UNSUPPORTED,
                         "layout ops are limited to tensors below 2^31 elements");
    unsigned grid = (unsigned)std::min<long long>((out_total + 255) / 256, 1 << 20);
    hipLaunchKernelGGL(chain_interp_kernel, dim3(grid), dim3(256), 0, as_stream(stream), x, y, cp,
                       (unsigned)out_total);
    return check_launch("chain_interp_kernel");
}

int pet_hip_split(const float *x, float *const *ys, int k, const int *in_dims, int rank, int dim,
                  const int *out_sizes, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (!dims_ok(in_dims, rank) || dim < 0 || dim >= rank || k < 1 || !ys || !out_sizes)
        return set_error(PET_HIP_ERR_INVALID, "bad split arguments");
    long long sum = 0;
    for (int i = 0; i < k; ++i) {
        if (out_sizes[i] < 0)
            return set_error(PET_HIP_ERR_INVALID, "negative split size");
        sum += out_sizes[i];
    }
    if (sum != in_dims[dim])
        return set_error(PET_HIP_ERR_INVALID, "split sizes sum to %lld, dim is %d", sum,
                         in_dims[dim]);
    long long istr[PET_HIP_MAX_RANK];
    row_major_strides(in_dims, rank, istr);
    long long in_total = prod(in_dims, rank);
    int off = 0;
    for (int i = 0; i < k; ++i) {
        int od[PET_HIP_MAX_RANK];
        for (int j = 0; j < rank; ++j)
            od[j] = in_dims[j];
        od[dim] = out_sizes[i];
        long long ostr[PET_HIP_MAX_RANK];
        row_major_strides(od, rank, ostr);
        ViewDesc v;
        v.rank = rank;
        v.obase = 0;
        v.ibase = (long long)off * istr[dim];
        for (int j = 0; j < rank; ++j)
            v.d[j] = plain_dim(od[j], ostr[j], istr[j]);
        int rc = launch_view_copy(x, ys[i], v, in_total, prod(od, rank), as_stream(stream));
        if (rc)
            return rc;
        off += out_sizes[i];
    }
    return PET_HIP_OK;
}

int pet_hip_concat(const float *const *xs, int k, float *y, const int *out_dims, int rank, int dim,
                   const int *in_sizes, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (!dims_ok(out_dims, rank) || dim < 0 || dim >= rank || k < 1 || !xs || !in_sizes)
        return set_error(PET_HIP_ERR_INVALID, "bad concat arguments");
    long long sum = 0;
    for (int i = 0; i < k; ++i) {
        if (in_sizes[i] < 0)
            return set_error(PET_HIP_ERR_INVALID, "negative concat size");
        sum += in_sizes[i];
    }
    if (sum != out_dims[dim])
        return set_error(PET_HIP_ERR_INVALID, "concat sizes sum to %lld, dim is %d", sum,
                         out_dims[dim]);
    long long ostr[PET_HIP_MAX_RANK];
    row_major_strides(out_dims, rank, ostr);
    long long out_total = prod(out_dims, rank);
    int off = 0;
    for (int i = 0; i < k; ++i) {
        int id[PET_HIP_MAX_RANK];
        for (int j = 0; j < rank; ++j)
            id[j] = out_dims[j];
        id[dim] = in_sizes[i];
        long long istr[PET_HIP_MAX_RANK];
        row_major_strides(id, rank, istr);
        ViewDesc v;
        v.rank = rank;
        v.ibase = 0;
        v.obase = (long long)off * ostr[dim];
        for (int j = 0; j < rank; ++j)
            v.d[j] = plain_dim(id[j], ostr[j], istr[j]);
        int rc = launch_view_copy(xs[i], y, v, prod(id, rank), out_total, as_stream(stream));
        if (rc)
            return rc;
        off += in_sizes[i];
    }
    return PET_HIP_OK;
}

int pet_hip_pad(const float *x, float *y, const int *in_dims, const int *begin, const int *end,
                int rank, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (!dims_ok(in_dims, rank) || !begin || !end)
        return set_error(PET_HIP_ERR_INVALID, "bad pad arguments");
    int od[PET_HIP_MAX_RANK];
    for (int i = 0; i < rank; ++i) {
        if (begin[i] < 0 || end[i] < 0)
            return set_error(PET_HIP_ERR_INVALID, "negative pad");
        od[i] = in_dims[i] + begin[i] + end[i];
    }
    long long istr[PET_HIP_MAX_RANK], ostr[PET_HIP_MAX_RANK];
    row_major_strides(in_dims, rank, istr);
    row_major_strides(od, rank, ostr);
    ViewDesc v;
    v.rank = rank;
    v.ibase = v.obase = 0;
    for (int j = 0; j < rank; ++j) {
        v.d[j] = plain_dim(od[j], ostr[j], istr[j]);
        v.d[j].lo = begin[j];
        v.d[j].hi = begin[j] + in_dims[j];
        v.ibase -= (long long)begin[j] * istr[j];
    }
    return launch_view_copy(x, y, v, prod(in_dims, rank), prod(od, rank), as_stream(stream));
}

int pet_hip_slice(const float *x, float *y, const int *in_dims, const int *begin, const int *end,
                  int rank, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (!dims_ok(in_dims, rank) || !begin || !end)
        return set_error(PET_HIP_ERR_INVALID, "bad slice arguments");
    int od[PET_HIP_MAX_RANK];
    for (int i = 0; i < rank; ++i) {
        if (begin[i] < 0 || end[i] < 0 || in_dims[i] < begin[i] + end[i])
            return set_error(PET_HIP_ERR_INVALID, "slice outside the tensor on dim %d", i);
        od[i] = in_dims[i] - begin[i] - end[i];
    }
    long long istr[PET_HIP_MAX_RANK], ostr[PET_HIP_MAX_RANK];
    row_major_strides(in_dims, rank, istr);
    row_major_strides(od, rank, ostr);
    ViewDesc v;
    v.rank = rank;
    v.ibase = v.obase = 0;
    for (int j = 0; j < rank; ++j) {
        v.d[j] = plain_dim(od[j], ostr[j], istr[j]);
        v.ibase += (long long)begin[j] * istr[j];
    }
    return launch_view_copy(x, y, v, prod(in_dims, rank), prod(od, rank), as_stream(stream));
}

int pet_hip_extend(const float *x, float *y, const int *in_dims, int rank, int dim, int num,
                   pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (!dims_ok(in_dims, rank) || dim < 0 || dim >= rank || num < 0)
        return set_error(PET_HIP_ERR_INVALID, "bad extend arguments");
    if (rank + 1 > PET_HIP_MAX_RANK)
        return set_error(PET_HIP_ERR_UNSUPPORTED, "extend supports rank <= %d",
                         PET_HIP_MAX_RANK - 1);
    // output viewed as [..., num+1, dims[dim], ...]: the repeat dim reads with stride 0
    long long istr[PET_HIP_MAX_RANK];
    row_major_strides(in_dims, rank, istr);
    int od[PET_HIP_MAX_RANK];
    long long isv[PET_HIP_MAX_RANK];
    int r = 0;
    for (int j = 0; j < rank; ++j) {
        if (j == dim) {
            od[r] = num + 1;
            isv[r++] = 0;
        }
        od[r] = in_dims[j];
        isv[r++] = istr[j];
    }
    long long ostr[PET_HIP_MAX_RANK];
    row_major_strides(od, r, ostr);
    ViewDesc v;
    v.rank = r;
    v.ibase = v.obase = 0;
    for (int j = 0; j < r; ++j)
        v.d[j] = plain_dim(od[j], ostr[j], isv[j]);
    return launch_view_copy(x, y, v, prod(in_dims, rank), prod(od, r), as_stream(stream));
}

} // extern "C"
